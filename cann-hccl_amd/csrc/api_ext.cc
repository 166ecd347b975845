// The calls of include/hccl/hccl_amd_ext.h: settings of a group, what the last collective issued, planning without a device.
#include <chrono>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <map>
#include <set>
#include <sstream>
#include <string>
#include <vector>

#include "api_internal.h"
#include "ranktable.h"

using namespace hcclamd;
using namespace hcclamd::api;

extern "C" {

// ---- extension ----------------------------------------------------------------------------------------

HcclResult HcclAmdSetParam(HcclComm comm, const char *key, const char *value)
{
    CHK_PTR(comm);
    CHK_PTR(key);
    CHK_PTR(value);
    Comm *c = AsComm(comm);
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    std::lock_guard<std::mutex> lock(c->group->m);
    GroupConfig &cfg = c->group->cfg;
    std::string k(key), v(value);
    if (k == "algo") {
        if (v == "ring") {
            cfg.algo = ALGO_RING;
        } else if (v == "mesh") {
            cfg.algo = ALGO_MESH;
        } else if (v == "rhd") {
            cfg.algo = ALGO_RHD;
        } else if (v == "pairwise") {
            cfg.algo = ALGO_PAIRWISE;   // all-to-all family: the flat schedule also over several servers; others: ring
        } else if (v == "star") {
            cfg.algo = ALGO_STAR;       // broadcast: the root hands every rank the whole buffer; others: as "auto" would not, ring
        } else if (v == "hd_blocks") {
            cfg.algo = ALGO_HD_BLOCKS;  // broadcast: halving-doubling over blocks of power-of-two sizes; others: ring
        } else if (v == "auto") {
            cfg.algo = -1;
        } else {
            return HCCL_E_PARA;
        }
    } else if (k == "servers") {
        long n = std::atol(value);
        if (n < 1 || uint32_t(n) > c->group->p || c->group->p % uint32_t(n) != 0) {
            return HCCL_E_PARA;
        }
        cfg.servers = uint32_t(n);
    } else if (k == "level0") {
        if (v == "mesh") {
            cfg.level0Rings = 0;
        } else if (v == "ring") {
            cfg.level0Rings = 1;
        } else if (v == "ring4") {
            cfg.level0Rings = 4;
        } else {
            return HCCL_E_PARA;
        }
    } else if (k == "step_sweep") {
        if (v == "forward") {
            cfg.stepSweep = 0;
        } else if (v == "alternate") {
            cfg.stepSweep = 1;
        } else {
            return HCCL_E_PARA;
        }
    } else if (k == "cache_entries") {
        long n = std::atol(value);
        if (n < 1 || n > (1 << 20)) {
            return HCCL_E_PARA;
        }
        cfg.cacheEntries = uint32_t(n);
    } else if (k == "nic_ranks") {
        // the ranks of an 8-rank ring (the devices of every server of 8) that own a network port: "all", or a
        // comma-separated list of 1, 2 or 4 of them
        uint32_t mask = 0;
        if (v != "all" && !v.empty()) {
            if (c->group->p % 8 != 0) {
                return HCCL_E_PARA;
            }
            std::stringstream in(v);
            std::string item;
            while (std::getline(in, item, ',')) {
                char *end = nullptr;
                long r = std::strtol(item.c_str(), &end, 10);
                if (item.empty() || *end != 0 || r < 0 || r > 7 || ((mask >> r) & 1u)) {
                    return HCCL_E_PARA;
                }
                mask |= 1u << r;
            }
            const int ports = __builtin_popcount(mask);
            if (ports != 1 && ports != 2 && ports != 4 && ports != 8) {
                return HCCL_E_PARA;
            }
            if (ports == 8) {
                mask = 0;
            }
        }
        cfg.nicMask = mask;
    } else if (k == "fused_stores") {
        if (v == "auto") {
            cfg.fusedStores = -1;
        } else if (v == "nt") {
            cfg.fusedStores = 0;
        } else if (v == "ordinary") {
            cfg.fusedStores = 1;
        } else {
            return HCCL_E_PARA;
        }
    } else if (k == "team_tiles") {
        long n = std::atol(value);
        if (n < 0 || n > long(kTeamTiles)) {
            return HCCL_E_PARA;
        }
        cfg.teamTiles = uint32_t(n);
    } else if (k == "team") {
        if (v == "auto") {
            cfg.team = -1;
        } else if (v == "0" || v == "1") {
            cfg.team = v == "1" ? 1 : 0;
        } else {
            return HCCL_E_PARA;
        }
    } else if (k == "step_stores") {
        if (v == "auto") {
            cfg.stepStores = -1;
        } else if (v == "nt") {
            cfg.stepStores = 0;
        } else if (v == "ordinary") {
            cfg.stepStores = 1;
        } else {
            return HCCL_E_PARA;
        }
    } else if (k == "deterministic") {
        cfg.deterministic = v != "0";
    } else if (k == "fuse") {
        cfg.fuse = v != "0";
    } else if (k == "graph") {
        cfg.graph = v != "0";
    } else if (k == "buffsize_mib") {
        long n = std::atol(value);
        if (n < 1) {
            return HCCL_E_PARA;
        }
        cfg.cclBytes = uint64_t(n) << 20;
    } else if (k == "buffsize_bytes") {
        long long n = std::atoll(value);
        if (n < 16) {
            return HCCL_E_PARA;
        }
        cfg.cclBytes = uint64_t(n);
    } else if (k == "align") {
        long n = std::atol(value);
        if (n < 1) {
            return HCCL_E_PARA;
        }
        cfg.align = uint64_t(n);
    } else if (k == "blocks_per_cu") {
        long n = std::atol(value);
        if (n < 0 || n > 64) {
            return HCCL_E_PARA;
        }
        cfg.blocksPerCu = uint32_t(n);
    } else if (k == "launch_cap_mib") {
        long n = v == "auto" ? -1 : std::atol(value);
        if (n < -1 || n > (1 << 20)) {
            return HCCL_E_PARA;
        }
        cfg.launchCapMiB = int32_t(n);
    } else if (k == "blocking_arrive") {
        cfg.blockingArrive = v != "0";
    } else if (k == "arrive_timeout_ms") {
        long n = std::atol(value);
        if (n < 1) {
            return HCCL_E_PARA;
        }
        cfg.arriveTimeoutMs = uint32_t(n);
    } else {
        return HCCL_E_PARA;
    }
    return HCCL_SUCCESS;
}

HcclResult HcclAmdGetLastOpInfo(HcclComm comm, HcclAmdOpInfo *info)
{
    CHK_PTR(comm);
    CHK_PTR(info);
    Comm *c = AsComm(comm);
    if (c == nullptr) {
        return HCCL_E_PARA;
    }
    std::lock_guard<std::mutex> lock(c->group->m);
    const OpInfo &o = c->group->lastInfo;
    info->coll = o.coll;
    info->algo = o.algo;
    info->fused = o.fused;
    info->graph = o.graph;
    info->cacheHit = o.cacheHit;
    info->launches = o.launches;
    info->bytesRead = o.bytesRead;
    info->bytesWritten = o.bytesWritten;
    info->schedRead = o.stepRead;
    info->schedWritten = o.stepWritten;
    info->scratchBytes = o.scratchBytes;
    info->teamLaunches = o.teamLaunches;
    info->reserved = 0;
    return HCCL_SUCCESS;
}

HcclResult HcclAmdDescribePlan(int32_t coll, int32_t algo, uint32_t nRanks, uint64_t count, HcclDataType dataType,
    uint64_t cclBytes, uint64_t align, uint64_t inPlaceMask, const uint64_t *tables, char *out, size_t cap, size_t *needed)
{
    CHK_PTR(out);
    if (nRanks == 0 || nRanks > kMaxRanks || !DataTypeKnown(dataType) || coll < 0 || coll > 6) {
        return HCCL_E_PARA;
    }
    PlanRequest rq;
    rq.coll = CollKind(coll);
    if (coll >= COLL_BROADCAST) {
        // rooted collectives: low 16 bits = root rank, bits 16..19 = schedule (0 ring, 1 mesh, 2 rhd, 4 mesh uncut, 5 star, 6 hd over blocks);
        // reduce only: bits 20..27 = number of rank groups of the two-level schedule, bit 28 = its mesh level uncut,
        // bit 29 / bit 30 = one ring / four rings inside a group instead of the mesh
        rq.root = uint32_t(algo) & 0xffffu;
        rq.algo = Algo((uint32_t(algo) >> 16) & 0xfu);
        if (coll == COLL_SCATTER) {
            rq.algo = ((uint32_t(algo) >> 20) & 1u) ? ALGO_RING : ALGO_MESH;   // scatter: bit 20 = the ring schedule
            rq.servers = std::max(1u, (uint32_t(algo) >> 21) & 0xffu);         // bits 21..28 = rank groups (two levels, mesh only)
            rq.level0Rings = ((uint32_t(algo) >> 29) & 1u) ? 1u : (((uint32_t(algo) >> 30) & 1u) ? 4u : 0u);   // as for the reduce
        }
        if (coll == COLL_BROADCAST) {
            rq.servers = std::max(1u, (uint32_t(algo) >> 20) & 0xffu);   // broadcast: bits 20..27 = rank groups (two levels)
            rq.level0Rings = ((uint32_t(algo) >> 29) & 1u) ? 1u : (((uint32_t(algo) >> 30) & 1u) ? 4u : 0u);   // as for the reduce
        }
        if (coll == COLL_REDUCE) {
            rq.servers = std::max(1u, (uint32_t(algo) >> 20) & 0xffu);
            rq.meshAtomic = ((uint32_t(algo) >> 28) & 1u) != 0;
            rq.level0Rings = ((uint32_t(algo) >> 29) & 1u) ? 1u : (((uint32_t(algo) >> 30) & 1u) ? 4u : 0u);   // bit 29 one ring, bit 30 four
        }
    } else if (coll == COLL_ALLREDUCE) {
        // all-reduce: low 8 bits = schedule, bits 8..15 = number of rank groups ("servers") of a two-level schedule
        rq.algo = Algo(uint32_t(algo) & 0xffu);
        rq.servers = std::max(1u, (uint32_t(algo) >> 8) & 0xffu);
        rq.meshAtomic = ((uint32_t(algo) >> 16) & 1u) != 0;   // bit 16: mesh level without the piece cut
        rq.level0Rings = (uint32_t(algo) >> 17) & 7u;         // bits 17..19: rings inside a group (0 = mesh, 1, 4)
        rq.nicMask = (uint32_t(algo) >> 20) & 0xffu;          // bits 20..27: ranks with a network port (8-rank ring)
    } else if (coll == COLL_REDUCESCATTER || coll == COLL_ALLGATHER) {
        // reduce-scatter, all-gather: the same fields
        rq.algo = Algo(uint32_t(algo) & 0xffu);
        rq.servers = std::max(1u, (uint32_t(algo) >> 8) & 0xffu);
        rq.meshAtomic = ((uint32_t(algo) >> 16) & 1u) != 0;
        rq.level0Rings = (uint32_t(algo) >> 17) & 7u;
        if (coll == COLL_REDUCESCATTER) {
            rq.nicMask = (uint32_t(algo) >> 20) & 0xffu;      // bits 20..27: devices of every server with a network port
        }
    } else if (coll == COLL_ALLTOALLV) {
        // all-to-all-v: bits 8..15 = number of servers of the staged schedule (0 or 1 = flat pairwise)
        rq.algo = ALGO_PAIRWISE;
        rq.servers = std::max(1u, (uint32_t(algo) >> 8) & 0xffu);
    } else {
        rq.algo = Algo(algo);
    }
    rq.p = nRanks;
    rq.count = count;
    rq.unit = ElemSize(dataType);
    rq.cclBytes = cclBytes;
    rq.align = align;
    rq.alias.assign(nRanks, 0);
    for (uint32_t r = 0; r < nRanks; r++) {
        rq.alias[r] = (inPlaceMask >> r) & 1ull;
    }
    if (coll == COLL_ALLTOALLV) {
        CHK_PTR(tables);
        size_t n = size_t(nRanks) * nRanks;
        rq.sendCounts.assign(tables, tables + n);
        rq.sdispls.assign(tables + n, tables + 2 * n);
        rq.recvCounts.assign(tables + 2 * n, tables + 3 * n);
        rq.rdispls.assign(tables + 3 * n, tables + 4 * n);
    }
    if ((coll == COLL_REDUCESCATTER || coll == COLL_ALLGATHER) && tables != nullptr) {
        rq.vCounts.assign(tables, tables + nRanks);
        rq.vDispls.assign(tables + nRanks, tables + 2 * size_t(nRanks));
    }
    Plan plan;
    std::string err;
    int rc = BuildPlan(rq, &plan, &err);
    if (rc != 0) {
        HCCL_LOG_ERROR("HcclAmdDescribePlan: %s", err.c_str());
        return rc == 1 ? HCCL_E_PARA : HCCL_E_INTERNAL;
    }
    std::string js = DescribePlan(plan);
    if (needed) {
        *needed = js.size() + 1;
    }
    if (js.size() + 1 > cap) {
        return HCCL_E_MEMORY;
    }
    std::memcpy(out, js.c_str(), js.size() + 1);
    return HCCL_SUCCESS;
}

}  // extern "C"

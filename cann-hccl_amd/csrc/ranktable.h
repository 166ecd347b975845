// Reads the part of a cluster rank table (the JSON file handed to HcclCommInitClusterInfo) that the
// single-GPU data path can use: which ranks exist and how they group into servers.
//
// Reference: FW/common/src/topo/topoinfo_ranktableConcise.cc:195-360 ("server_count", "server_list",
// per server "server_id" and "device": [{"device_id", "rank_id", ...}]); addresses, ports and super-pod
// entries are accepted and ignored (FW = src/domain/collective_communication/framework).
#pragma once
#include <cstdint>
#include <string>
#include <vector>

namespace hcclamd {

struct RankTableServer {
    std::string id;
    std::vector<uint32_t> ranks;     // rank_id of every device entry, in file order
    std::vector<uint32_t> devices;   // device_id of every device entry
};

struct RankTable {
    std::vector<RankTableServer> servers;
    uint32_t rankCount = 0;
};

// Returns 0 on success; 1 when the text is not a usable rank table (`err` says why).
int ParseRankTable(const std::string &text, RankTable *out, std::string *err);

}  // namespace hcclamd

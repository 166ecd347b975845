#include "ranktable.h"

#include <cctype>
#include <cstdlib>
#include <map>
#include <memory>
#include <set>

namespace hcclamd {
namespace {

// A JSON value, just enough structure for the rank table.
struct Json {
    enum Kind { NUL, BOOL, NUM, STR, ARR, OBJ } kind = NUL;
    std::string text;                                  // STR: the string; NUM / BOOL: the literal
    std::vector<Json> items;                           // ARR
    std::vector<std::pair<std::string, Json>> fields;  // OBJ, in file order

    const Json *Get(const std::string &key) const
    {
        for (const auto &f : fields) {
            if (f.first == key) {
                return &f.second;
            }
        }
        return nullptr;
    }
};

struct Parser {
    const std::string &s;
    size_t at = 0;
    std::string err;
    int depth = 0;

    explicit Parser(const std::string &text) : s(text) {}

    void Skip()
    {
        while (at < s.size() && std::isspace(static_cast<unsigned char>(s[at]))) {
            at++;
        }
    }
    bool Fail(const char *what)
    {
        if (err.empty()) {
            err = std::string(what) + " at byte " + std::to_string(at);
        }
        return false;
    }
    bool String(std::string *out)
    {
        if (at >= s.size() || s[at] != '"') {
            return Fail("expected a string");
        }
        at++;
        out->clear();
        while (at < s.size() && s[at] != '"') {
            char c = s[at++];
            if (c == '\\') {
                if (at >= s.size()) {
                    return Fail("unterminated escape");
                }
                char e = s[at++];
                switch (e) {
                    case 'n': out->push_back('\n'); break;
                    case 't': out->push_back('\t'); break;
                    case 'r': out->push_back('\r'); break;
                    case 'b': out->push_back('\b'); break;
                    case 'f': out->push_back('\f'); break;
                    case 'u':
                        if (at + 4 > s.size()) {
                            return Fail("short \\u escape");
                        }
                        out->push_back('?');   // code points are of no interest here
                        at += 4;
                        break;
                    default: out->push_back(e); break;   // \" \\ \/
                }
            } else {
                out->push_back(c);
            }
        }
        if (at >= s.size()) {
            return Fail("unterminated string");
        }
        at++;
        return true;
    }
    bool Value(Json *v)
    {
        if (++depth > 64) {
            return Fail("nesting too deep");
        }
        Skip();
        if (at >= s.size()) {
            return Fail("unexpected end");
        }
        bool ok = true;
        char c = s[at];
        if (c == '{') {
            v->kind = Json::OBJ;
            at++;
            Skip();
            if (at < s.size() && s[at] == '}') {
                at++;
            } else {
                for (;;) {
                    Skip();
                    std::string key;
                    Json val;
                    if (!String(&key)) {
                        return false;
                    }
                    Skip();
                    if (at >= s.size() || s[at] != ':') {
                        return Fail("expected ':'");
                    }
                    at++;
                    if (!Value(&val)) {
                        return false;
                    }
                    v->fields.emplace_back(std::move(key), std::move(val));
                    Skip();
                    if (at < s.size() && s[at] == ',') {
                        at++;
                        continue;
                    }
                    if (at < s.size() && s[at] == '}') {
                        at++;
                        break;
                    }
                    return Fail("expected ',' or '}'");
                }
            }
        } else if (c == '[') {
            v->kind = Json::ARR;
            at++;
            Skip();
            if (at < s.size() && s[at] == ']') {
                at++;
            } else {
                for (;;) {
                    Json val;
                    if (!Value(&val)) {
                        return false;
                    }
                    v->items.push_back(std::move(val));
                    Skip();
                    if (at < s.size() && s[at] == ',') {
                        at++;
                        continue;
                    }
                    if (at < s.size() && s[at] == ']') {
                        at++;
                        break;
                    }
                    return Fail("expected ',' or ']'");
                }
            }
        } else if (c == '"') {
            v->kind = Json::STR;
            ok = String(&v->text);
        } else {
            size_t b = at;
            while (at < s.size() && (std::isalnum(static_cast<unsigned char>(s[at])) || s[at] == '-' || s[at] == '+' || s[at] == '.')) {
                at++;
            }
            if (at == b) {
                return Fail("unexpected character");
            }
            v->text = s.substr(b, at - b);
            if (v->text == "null") {
                v->kind = Json::NUL;
            } else if (v->text == "true" || v->text == "false") {
                v->kind = Json::BOOL;
            } else {
                v->kind = Json::NUM;
            }
        }
        depth--;
        return ok;
    }
};

// The rank table writes numbers as strings ("rank_id": "3"); plain numbers are taken too.
bool AsUnsigned(const Json *v, uint32_t *out)
{
    if (v == nullptr || (v->kind != Json::STR && v->kind != Json::NUM) || v->text.empty()) {
        return false;
    }
    for (char c : v->text) {
        if (!std::isdigit(static_cast<unsigned char>(c))) {
            return false;
        }
    }
    if (v->text.size() > 9) {
        return false;
    }
    *out = static_cast<uint32_t>(std::strtoul(v->text.c_str(), nullptr, 10));
    return true;
}

}  // namespace

int ParseRankTable(const std::string &text, RankTable *out, std::string *err)
{
    Parser p(text);
    Json root;
    if (!p.Value(&root)) {
        *err = "rank table is not valid JSON: " + p.err;
        return 1;
    }
    p.Skip();
    if (p.at != text.size() || root.kind != Json::OBJ) {
        *err = "rank table must be one JSON object";
        return 1;
    }
    const Json *list = root.Get("server_list");
    if (list == nullptr || list->kind != Json::ARR) {
        *err = "rank table has no 'server_list'";
        return 1;
    }
    if (list->items.empty()) {
        *err = "the 'server_list' in the rank table is empty";
        return 1;
    }
    if (const Json *count = root.Get("server_count")) {
        uint32_t n = 0;
        if (!AsUnsigned(count, &n) || n != list->items.size()) {
            *err = "the 'server_count' in the rank table does not match 'server_list'";
            return 1;
        }
    }
    out->servers.clear();
    std::set<std::string> ids;
    std::set<uint32_t> ranks;
    for (const Json &srv : list->items) {
        const Json *id = srv.kind == Json::OBJ ? srv.Get("server_id") : nullptr;
        if (id == nullptr || id->kind != Json::STR || id->text.empty()) {
            *err = "a server entry has no 'server_id'";
            return 1;
        }
        if (!ids.insert(id->text).second) {
            *err = "server_id '" + id->text + "' appears twice";
            return 1;
        }
        const Json *dev = srv.Get("device");
        if (dev == nullptr || dev->kind != Json::ARR || dev->items.empty()) {
            *err = "server '" + id->text + "' has no devices";
            return 1;
        }
        RankTableServer s;
        s.id = id->text;
        for (const Json &d : dev->items) {
            uint32_t rank = 0, device = 0;
            if (d.kind != Json::OBJ || !AsUnsigned(d.Get("rank_id"), &rank) || !AsUnsigned(d.Get("device_id"), &device)) {
                *err = "a device entry of server '" + id->text + "' lacks 'rank_id' or 'device_id'";
                return 1;
            }
            if (!ranks.insert(rank).second) {
                *err = "rank_id " + std::to_string(rank) + " appears twice";
                return 1;
            }
            s.ranks.push_back(rank);
            s.devices.push_back(device);
        }
        out->servers.push_back(std::move(s));
    }
    out->rankCount = static_cast<uint32_t>(ranks.size());
    if (*ranks.rbegin() != out->rankCount - 1) {
        *err = "rank ids must be 0 .. n-1";
        return 1;
    }
    return 0;
}

}  // namespace hcclamd

// engine/registry.cpp -- the family registry of sequence_model.h
#include "sequence_model.h"
#include "safetensors.h"
#include "../../../include/ntk.h"

#include <map>

namespace nt {

static std::map<std::string, FamilyFactory>& table() {
    static std::map<std::string, FamilyFactory> t;   // built on first use: registrars run during static initialisation
    return t;
}

FamilyRegistrar::FamilyRegistrar(const char* architecture, FamilyFactory make) { table()[architecture] = std::move(make); }

std::vector<std::string> registered_families() {
    std::vector<std::string> out;
    for (const auto& kv : table()) out.push_back(kv.first);
    return out;
}

std::unique_ptr<SequenceModel> make_family(const std::string& architecture) {
    auto it = table().find(architecture);
    if (it == table().end()) return nullptr;
    return it->second();
}

std::unique_ptr<SequenceModel> open_model(const std::string& path, const SeqLoadOptions& opt, std::string* why) {
    auto fail = [&](const std::string& s) { if (why) *why = s; return std::unique_ptr<SequenceModel>(); };
    if (!ModelFolder::looks_like(path)) return fail(path + " is not a model folder (no config.json)");
    const std::string arch = ModelFolder::architecture_of(path);
    if (arch.empty()) return fail(path + "/config.json names no architecture");
    auto m = make_family(arch);
    if (!m) {
        std::string have;
        for (const auto& f : registered_families()) have += (have.empty() ? "" : ", ") + f;
        return fail("no model family for architecture '" + arch + "' (have: " + have + ")");
    }
    const int st = m->load(path, opt);
    if (st != NTK_OK) return fail(m->error().empty() ? std::string(ntk_status_string(st)) : m->error());
    return m;
}

}  // namespace nt

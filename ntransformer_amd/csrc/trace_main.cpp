// trace_main.cpp -- `trace_run`: replays a token trace through a model folder and writes logits; it samples nothing.
//
//   trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N
//
// Standard input: one JSON object per line, {"step": k, "entries": [{"id": "...", "tokens": [...], "want": [...]}, ...], "end": ["...", ...]}.
// Every entry appends its tokens to the request's slot of the model's cache (a new id takes a free slot) through SequenceModel::forward -- the
// step function generation uses; the logits of the places in "want" go to OUT/<step>.f32 as little-endian F32 [wanted][vocab], in the order of the
// entries; the requests in "end" give their slots back; then "done <step>" is printed and flushed.  End of input: exit 0.
// The model class is chosen by config.json's "architecture" through the family registry.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <iostream>
#include <map>
#include <string>
#include <vector>
#include "engine/json.h"
#include "engine/sequence_model.h"
#include "../../include/ntk.h"

int main(int argc, char** argv) {
    std::string model, dtype = "bfloat16", out;
    int max_tokens = 4096;
    for (int i = 1; i < argc; ++i) {
        const std::string a = argv[i];
        auto val = [&]() -> const char* { return i + 1 < argc ? argv[++i] : ""; };
        if (a == "--model") model = val();
        else if (a == "--dtype") dtype = val();
        else if (a == "--out") out = val();
        else if (a == "--max-tokens") max_tokens = atoi(val());
        else if (a == "-h" || a == "--help") {
            printf("usage: %s --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N  < steps.jsonl\n", argv[0]);
            return 0;
        } else { fprintf(stderr, "unknown option %s\n", a.c_str()); return 2; }
    }
    if (model.empty() || out.empty()) { fprintf(stderr, "--model and --out are required\n"); return 2; }
    if (dtype != "bfloat16" && dtype != "float32") { fprintf(stderr, "--dtype must be bfloat16 or float32\n"); return 2; }
    if (max_tokens < 1) max_tokens = 1;
    nt::SeqLoadOptions opt;
    opt.max_context = max_tokens;   // one request may hold all of them
    opt.slots = 4;                  // requests normally come one after the other; a few may overlap
    opt.float32 = dtype == "float32";
    std::string why;
    std::unique_ptr<nt::SequenceModel> m = nt::open_model(model, opt, &why);
    if (!m) { fprintf(stderr, "cannot load %s: %s\n", model.c_str(), why.c_str()); return 1; }
    const int V = m->info().vocab;
    std::map<std::string, int> slot_of;
    std::string line;
    std::vector<float> rows;
    while (std::getline(std::cin, line)) {
        if (line.find_first_not_of(" \t\r\n") == std::string::npos) continue;
        nt::Json j;
        if (!j.parse(line.data(), line.size()) || !j.is_object()) { fprintf(stderr, "a step is not a JSON object\n"); return 1; }
        const long long step = j.at("step").integer();
        std::vector<float> wanted;
        for (const nt::Json& e : j.at("entries").arr) {
            const std::string id = e.at("id").str;
            std::vector<int> tokens, want;
            for (const auto& t : e.at("tokens").arr) tokens.push_back((int)t.integer());
            for (const auto& w : e.at("want").arr) want.push_back((int)w.integer());
            auto it = slot_of.find(id);
            if (it == slot_of.end()) {
                const int s = m->acquire_slot();
                if (s < 0) { fprintf(stderr, "no free slot for request %s\n", id.c_str()); return 1; }
                it = slot_of.emplace(id, s).first;
            }
            if (tokens.empty()) continue;
            if (!m->forward(it->second, tokens.data(), (int)tokens.size(), want.data(), (int)want.size())) {
                fprintf(stderr, "step %lld failed: %s\n", step, m->error().c_str());
                return 1;
            }
            if (!want.empty()) {
                rows.resize(want.size() * (size_t)V);
                if (m->copy_logits(rows.data(), (int)want.size()) != NTK_OK) { fprintf(stderr, "step %lld: copying the logits failed\n", step); return 1; }
                wanted.insert(wanted.end(), rows.begin(), rows.end());
            }
        }
        if (m->sync() != NTK_OK) { fprintf(stderr, "step %lld: the device reported an error\n", step); return 1; }
        if (!wanted.empty()) {
            const std::string path = out + "/" + std::to_string(step) + ".f32";
            FILE* f = fopen(path.c_str(), "wb");
            if (!f || fwrite(wanted.data(), sizeof(float), wanted.size(), f) != wanted.size()) { fprintf(stderr, "cannot write %s\n", path.c_str()); return 1; }
            fclose(f);
        }
        for (const nt::Json& e : j.at("end").arr) {
            auto it = slot_of.find(e.str);
            if (it != slot_of.end()) { m->release_slot(it->second); slot_of.erase(it); }
        }
        printf("done %lld\n", step);
        fflush(stdout);
    }
    return 0;
}

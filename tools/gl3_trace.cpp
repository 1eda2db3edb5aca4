// gl3_trace — replays a trace of steps through a plan, one JSON object per line on standard input:
//     {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
// Every entry carries the next tokens of a request; a request seen for the first time takes a free sequence slot (gl3_seq_acquire) and
// starts at position 0, later entries continue where the request stopped (gl3_forward_step runs only the new tokens, from the slot's
// cache and state); "end" gives the slots back.  For a step with wanted rows the logits are written to <out>/<step>.f32 as little-endian
// float32 [wanted][vocab], in the order of the entries and of "want"; after every step "done <step>" is printed.  Nothing is sampled.
//
//   gl3_trace --model DIR|file.gguf --dtype bfloat16|float32 --out DIR [--max-tokens N] [--batch B] [--slots S]
// Model folders (config.json + model.safetensors) load through gl3_load_model_dir; --dtype float32 widens the matrices and runs every
// product in float32.  Exit codes: 0 end of input, 2 usage, 3 float32 asked of a model that has no float32 plan, 1 anything else.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <iostream>
#include <map>
#include <string>
#include <vector>

#include "../include/gpullama3_hip.h"

struct Entry { std::string id; std::vector<int32_t> tokens, want; };
struct Step { long step = -1; std::vector<Entry> entries; std::vector<std::string> end; };

// reader for the line format above (objects, arrays, strings without escapes beyond \" and \\, integers)
struct Reader {
    const char* p;
    void ws() { while (*p == ' ' || *p == '\t' || *p == '\r' || *p == '\n') ++p; }
    bool lit(char c) { ws(); if (*p != c) return false; ++p; return true; }
    bool str(std::string& out) {
        ws();
        if (*p != '"') return false;
        ++p; out.clear();
        while (*p && *p != '"') { if (*p == '\\' && p[1]) ++p; out += *p++; }
        if (*p != '"') return false;
        ++p;
        return true;
    }
    bool num(long& v) { ws(); char* e; v = strtol(p, &e, 10); if (e == p) return false; p = e; return true; }
    bool ints(std::vector<int32_t>& out) {
        if (!lit('[')) return false;
        if (lit(']')) return true;
        do { long v; if (!num(v)) return false; out.push_back((int32_t)v); } while (lit(','));
        return lit(']');
    }
    bool strs(std::vector<std::string>& out) {
        if (!lit('[')) return false;
        if (lit(']')) return true;
        do { std::string s; if (!str(s)) return false; out.push_back(s); } while (lit(','));
        return lit(']');
    }
    bool skip() {          // any value
        ws();
        if (*p == '"') { std::string s; return str(s); }
        if (*p == '{' || *p == '[') {
            const char open = *p, close = open == '{' ? '}' : ']';
            ++p;
            if (lit(close)) return true;
            do { if (open == '{') { std::string k; if (!str(k) || !lit(':')) return false; } if (!skip()) return false; } while (lit(','));
            return lit(close);
        }
        while (*p && !strchr(",}] \t\r\n", *p)) ++p;
        return true;
    }
    bool entry(Entry& e) {
        if (!lit('{')) return false;
        if (lit('}')) return true;
        do {
            std::string k;
            if (!str(k) || !lit(':')) return false;
            if (k == "id") { if (!str(e.id)) return false; }
            else if (k == "tokens") { if (!ints(e.tokens)) return false; }
            else if (k == "want") { if (!ints(e.want)) return false; }
            else if (!skip()) return false;
        } while (lit(','));
        return lit('}');
    }
    bool step(Step& s) {
        if (!lit('{')) return false;
        if (lit('}')) return true;
        do {
            std::string k;
            if (!str(k) || !lit(':')) return false;
            if (k == "step") { if (!num(s.step)) return false; }
            else if (k == "entries") {
                if (!lit('[')) return false;
                if (!lit(']')) {
                    do { s.entries.emplace_back(); if (!entry(s.entries.back())) return false; } while (lit(','));
                    if (!lit(']')) return false;
                }
            } else if (k == "end") { if (!strs(s.end)) return false; }
            else if (!skip()) return false;
        } while (lit(','));
        return lit('}');
    }
};

int main(int argc, char** argv) {
    std::string model, dtype = "bfloat16", out;
    long max_tokens = 0, batch = 512, slots = 4;
    for (int i = 1; i < argc; ++i) {
        const std::string a = argv[i];
        auto val = [&]() -> const char* { if (i + 1 >= argc) { fprintf(stderr, "gl3_trace: %s needs a value\n", a.c_str()); exit(2); } return argv[++i]; };
        if (a == "--model") model = val();
        else if (a == "--dtype") dtype = val();
        else if (a == "--out") out = val();
        else if (a == "--max-tokens") max_tokens = atol(val());
        else if (a == "--batch") batch = atol(val());
        else if (a == "--slots") slots = atol(val());
        else { fprintf(stderr, "gl3_trace: unknown option %s\n", a.c_str()); return 2; }
    }
    if (model.empty() || out.empty() || (dtype != "bfloat16" && dtype != "float32") || batch < 1 || slots < 1) {
        fprintf(stderr, "usage: gl3_trace --model DIR --dtype bfloat16|float32 --out DIR [--max-tokens N] [--batch B] [--slots S]\n");
        return 2;
    }
    gl3_model_desc opts{};
    opts.struct_size = sizeof opts;
    opts.ctx = max_tokens > 0 ? (int32_t)max_tokens : 0;
    opts.max_batch = (int32_t)batch;
    opts.n_seqs = (int32_t)slots;
    gl3_ctx* ctx = nullptr;
    int32_t r;
    if (gl3_is_model_dir(model.c_str())) {
        if (dtype == "float32") opts.flags |= GL3_FLAG_F32_COMPUTE;
        r = gl3_load_model_dir(model.c_str(), &opts, &ctx);
    } else {
        if (dtype == "float32") { fprintf(stderr, "gl3_trace: GGUF plans have no float32 matrices\n"); return 3; }
        opts.n_seqs = 1;
        r = gl3_load_gguf(model.c_str(), &opts, &ctx);
    }
    if (r != GL3_OK) { fprintf(stderr, "gl3_trace: loading %s failed (%d): %s\n", model.c_str(), r, gl3_last_error(nullptr)); return 1; }
    gl3_model_desc d{};
    gl3_get_model_desc(ctx, &d);
    const size_t V = (size_t)d.vocab;

    struct Live { int32_t slot; int32_t pos; };
    std::map<std::string, Live> live;
    std::string line;
    std::vector<float> logits;
    while (std::getline(std::cin, line)) {
        if (line.find_first_not_of(" \t\r\n") == std::string::npos) continue;
        Step s;
        Reader rd{line.c_str()};
        if (!rd.step(s) || s.step < 0) { fprintf(stderr, "gl3_trace: cannot read step: %.200s\n", line.c_str()); gl3_destroy(ctx); return 1; }
        size_t rows = 0;
        for (auto& e : s.entries) rows += e.want.size();
        logits.resize(rows * V);
        size_t row = 0;
        for (auto& e : s.entries) {
            auto it = live.find(e.id);
            if (it == live.end()) {
                int32_t slot = -1;
                if ((r = gl3_seq_acquire(ctx, &slot)) != GL3_OK) { fprintf(stderr, "gl3_trace: step %ld: %s\n", s.step, gl3_last_error(ctx)); gl3_destroy(ctx); return 1; }
                it = live.emplace(e.id, Live{slot, 0}).first;
            }
            if (e.tokens.empty()) continue;
            r = gl3_forward_step(ctx, it->second.slot, e.tokens.data(), (int32_t)e.tokens.size(), it->second.pos, e.want.data(), (int32_t)e.want.size(),
                                 e.want.empty() ? nullptr : logits.data() + row * V);
            if (r != GL3_OK) { fprintf(stderr, "gl3_trace: step %ld, request %s: %s\n", s.step, e.id.c_str(), gl3_last_error(ctx)); gl3_destroy(ctx); return 1; }
            it->second.pos += (int32_t)e.tokens.size();
            row += e.want.size();
        }
        if (rows) {
            const std::string path = out + "/" + std::to_string(s.step) + ".f32";
            FILE* f = fopen(path.c_str(), "wb");
            if (!f || fwrite(logits.data(), 4, logits.size(), f) != logits.size() || fclose(f) != 0) { fprintf(stderr, "gl3_trace: cannot write %s\n", path.c_str()); gl3_destroy(ctx); return 1; }
        }
        for (auto& id : s.end) {
            auto it = live.find(id);
            if (it != live.end()) { gl3_seq_release(ctx, it->second.slot); live.erase(it); }
        }
        printf("done %ld\n", s.step);
        fflush(stdout);
    }
    gl3_destroy(ctx);
    return 0;
}

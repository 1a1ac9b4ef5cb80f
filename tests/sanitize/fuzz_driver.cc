// Fuzz driver for the host-only part of the library (graph loader, linker, trigger round trip,
// fused-step grouping), built by tests/test_host_sanitizers.py with AddressSanitizer and
// UndefinedBehaviorSanitizer from graph.cc and program.cc directly: no HIP, no GPU.
// argv: pairs "<path stem of a golden graph> <world>", then optionally "--trials N".
// Every document is loaded and linked clean (three item sizes), then damaged N times (truncated,
// bytes overwritten, ranges deleted, numbers replaced by out-of-range ones) and loaded and linked
// again: errors must come back as pccl_hip::Error, and the sanitizers must stay silent.
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <random>
#include <sstream>
#include <string>
#include <vector>
#include "graph.h"
#include "program.h"
using namespace pccl_hip;
static std::string slurp(const std::string& p) { std::ifstream f(p, std::ios::binary); std::stringstream ss; ss << f.rdbuf(); return ss.str(); }
int main(int argc, char** argv) {
    int trials = 300;
    for (int a = 1; a + 1 < argc; ++a)
        if (std::string(argv[a]) == "--trials") { trials = atoi(argv[a + 1]); argc = a; break; }
    std::mt19937 rng(5);
    long loaded = 0, failed = 0, linked = 0, linkfail = 0;
    for (int a = 1; a + 1 < argc; a += 2) {
        std::string stem = argv[a]; int world = atoi(argv[a + 1]);
        std::vector<std::string> texts;
        for (int r = 0; r < world; ++r) texts.push_back(slurp(stem + "_rank" + std::to_string(r) + ".json"));
        // clean link
        try {
            std::vector<RankGraph> gs;
            for (auto& t : texts) gs.push_back(load_graph_json(t.data(), t.size()));
            std::vector<const RankGraph*> ps; for (auto& g : gs) ps.push_back(&g);
            for (int64_t tb : {0, 4096, 32768}) {
                LinkOptions opt; opt.step_tile_bytes = tb;
                Program P = link_program(ps, opt);
                std::vector<pccl_trigger> tr; std::vector<pccl_primitive_meta> me;
                graph_to_triggers(gs[0], &tr, &me);
                RankGraph back = graph_from_triggers(tr.data(), me.data(), (int)tr.size(), gs[0].collective_type.c_str());
                std::vector<pccl_fused_step> st; std::vector<int> off;
                build_fused_steps(gs[0], &st, &off);
                ++linked;
            }
        } catch (const Error& e) { printf("clean link of %s: %s\n", stem.c_str(), e.msg.c_str()); }
        for (int trial = 0; trial < trials; ++trial) {
            std::vector<std::string> mt = texts;
            int which = rng() % world;
            std::string& b = mt[which];
            int kind = rng() % 4;
            if (kind == 0) b.resize(rng() % b.size());
            else if (kind == 1) { for (int k = 0; k < 1 + (int)(rng() % 5); ++k) b[rng() % b.size()] = (char)(rng() % 256); }
            else if (kind == 2) { size_t i = rng() % b.size(); b.erase(i, 1 + rng() % 40); }
            else {
                // replace a digit run
                size_t i = rng() % b.size();
                while (i < b.size() && !(b[i] >= '0' && b[i] <= '9')) ++i;
                if (i < b.size()) { size_t j = i; while (j < b.size() && b[j] >= '0' && b[j] <= '9') ++j;
                    const char* reps[] = {"-1", "99999999999999999999", "2147483648", "1e9", "0.5", "9223372036854775807", "7", "3"};
                    b.replace(i, j - i, reps[rng() % 8]); }
            }
            try {
                std::vector<RankGraph> gs;
                for (auto& t : mt) gs.push_back(load_graph_json(t.data(), t.size()));
                ++loaded;
                std::vector<const RankGraph*> ps; for (auto& g : gs) ps.push_back(&g);
                try { Program P = link_program(ps, LinkOptions{}); ++linked; } catch (const Error&) { ++linkfail; }
            } catch (const Error&) { ++failed; }
        }
    }
    printf("loaded %ld failed %ld linked %ld linkfail %ld\n", loaded, failed, linked, linkfail);
    return 0;
}

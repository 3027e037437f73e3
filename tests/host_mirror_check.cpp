// A host-only program over the C++ mirror of the reference's operator API (qwen3.8-flash-next-2x-p100_amd/host/fnx.hpp):
// compiled and run by tests/test_host_mirror.py. It calls only functions that need no GPU (prompt lookup, acceptance,
// the sampler's distribution and draw, the GGUF reader) and prints what they return, one value a line.
#include <cstdio>
#include <cstdlib>

#include "../qwen3.8-flash-next-2x-p100_amd/host/fnx.hpp"

int main(int argc, char** argv) {
    try {
        // session.hpp:55-57: the tokens after the latest earlier place of the context's last three
        const std::vector<int> ctx = {5, 6, 7, 8, 9, 1, 2, 5, 6, 7};
        int match = -2;
        const std::vector<int> d = fnx::lookup_drafts(ctx, 4, 8, &match);
        std::printf("drafts %zu match %d first %d\n", d.size(), match, d.empty() ? -1 : d[0]);
        std::printf("accept %d\n", fnx::accept_greedy({9, 4, 5, 6}, {4, 5, 7, 1}));
        fnx::Sampling s;
        s.top_k = 2;
        const fnx::Dist dist = fnx::make_dist({{1.0f, 11}, {0.0f, 12}, {-1.0f, 13}}, s);
        std::printf("dist %zu p0 %.6f draw %d %d\n", dist.ids.size(), dist.p[0], fnx::draw(dist, 0.1), fnx::draw(dist, 0.9));
        if (argc > 1) {
            const fnx::Gguf g(argv[1]);
            const fnx_gguf_tensor t = g.t("w");
            std::printf("gguf tensors %d ne0 %lld arch %s\n", g.count(), (long long) t.ne[0], g.s("general.architecture").c_str());
            try {
                g.t("missing");
            } catch (const std::runtime_error& e) {
                std::printf("refused: %s\n", e.what());
            }
        }
    } catch (const std::exception& e) {
        std::printf("FAILED: %s\n", e.what());
        return 1;
    }
    return 0;
}

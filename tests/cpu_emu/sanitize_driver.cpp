// TEST INFRASTRUCTURE: a plain C++ program on the C ABI of the CPU-emulated engine, meant to be compiled together with
// the kernel sources under -fsanitize=address,undefined (tests/cpu_emu/build_emu.py: build_sanitize_driver).  It runs a
// few small seeded problems -- one tree and two, 1 to 6 dimensions, several columns, variance compression, the
// transposed product -- so that an access outside an array or undefined arithmetic in a kernel stops the program with a
// report.  Usage: sanitize_driver <first case> <number of cases> [points [dimension nodes min_points small_field_points]]
// (the last four replace what the case number would choose: e.g. 4 81 8 2 with 20000 points is a 4-D tree of three
// levels on the 3^4 grid, whose M2L takes the cells that all siblings list first).
#include "../../include/f3m.h"

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

int main(int argc, char **argv)
{
    const int first = argc > 1 ? atoi(argv[1]) : 0, ncase = argc > 2 ? atoi(argv[2]) : 8;
    const long long base = argc > 3 ? atoll(argv[3]) : 400;
    int failures = 0;
    for (int cs = first; cs < first + ncase; cs++) {
        std::mt19937 g(100 + cs);
        std::uniform_real_distribution<float> U(0.f, 1.f);
        std::normal_distribution<float> Nn(0.f, 1.f);
        const int dims[] = {1, 2, 3, 3, 4, 5, 6, 3};
        const int nodes_by_d[] = {0, 8, 16, 27, 16, 32, 64};
        const int d = argc > 7 ? atoi(argv[4]) : dims[cs % 8];
        const bool two = (cs % 3) == 1;
        const long long N = base + (long long)(g() % (unsigned)base), M = two ? base / 2 + (long long)(g() % (unsigned)base) : N;
        const int c = 1 + (cs % 4);
        f3m_params p{};
        p.ls = 0.2f + 2.f * U(g);
        p.min_points = (cs % 2) ? 40.f : 100.f;
        p.nr_of_interpolation = (cs % 5 == 4 && d == 3) ? 64 : nodes_by_d[d];
        p.var_compression = (cs % 4) == 3;
        p.eff_var_limit = 0.3f;
        p.small_field_points = 5 + (int)(g() % 30);
        if (argc > 7) {
            p.nr_of_interpolation = atoi(argv[5]);
            p.min_points = (float)atof(argv[6]);
            p.small_field_points = atoi(argv[7]);
            p.ls = 0.6f;
        }
        std::vector<float> X((size_t)N * d), Y((size_t)M * d), b((size_t)M * c), out((size_t)N * c), out2((size_t)N * c),
            u((size_t)N), outT((size_t)M);
        const bool normal = cs % 2;
        for (auto &v : X) v = normal ? Nn(g) : U(g);
        for (auto &v : Y) v = normal ? Nn(g) * 0.8f : U(g) * 1.1f;
        for (auto &v : b) v = Nn(g);
        for (auto &v : u) v = Nn(g);
        printf("case %d: d=%d N=%lld M=%lld columns=%d nodes=%d var_compression=%d trees=%d\n", cs, d, N, M, c,
               p.nr_of_interpolation, p.var_compression, two ? 2 : 1);
        fflush(stdout);
        const float *Yp = two ? Y.data() : nullptr;
        if (f3m_kmvm_f32(d, X.data(), N, Yp, M, b.data(), c, &p, out.data(), nullptr)) {
            printf("  product failed: %s\n", f3m_last_error());
            failures++;
            continue;
        }
        f3m_plan *plan = nullptr;
        if (f3m_plan_create(d, X.data(), N, Yp, M, &p, nullptr, &plan) || f3m_plan_apply(plan, b.data(), c, out2.data(), nullptr)) {
            printf("  plan failed: %s\n", f3m_last_error());
            failures++;
            continue;
        }
        bool same = true;
        for (size_t i = 0; i < out.size(); i++) same = same && out[i] == out2[i] && std::isfinite(out[i]);
        if (two && f3m_plan_apply_transpose(plan, u.data(), 1, outT.data(), nullptr)) {
            printf("  transposed product failed: %s\n", f3m_last_error());
            failures++;
        }
        printf("  depth %d, one-shot product and plan + apply %s\n", f3m_plan_depth(plan), same ? "agree bit for bit" : "DIFFER");
        if (!same) failures++;
        f3m_plan_destroy(plan);
    }
    f3m_release_cache();
    printf("%s\n", failures ? "FAILED" : "done");
    return failures ? 1 : 0;
}

/* A plain C program on the C ABI of include/f3m.h: device memory from the HIP runtime, no Python, no torch.
 * It multiplies a Gaussian kernel matrix of 60000 seeded points in three dimensions by two vectors through
 * f3m_kmvm_f32 and through a plan (forward and transposed), and compares with the exact products of
 * f3m_exact_f32.  Prints the relative L2 errors and "OK", or the library's error message.
 * Built by tests/abi_c/build_smoke.py; run by tests/test_gpu_parity.py::test_c_program_on_the_abi. */
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>

#include "f3m.h"

#define CHECK_HIP(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); return 2; } } while (0)
#define CHECK_F3M(x) do { int rc_ = (x); if (rc_ != 0) { printf("f3m error %d: %s (line %d)\n", rc_, f3m_last_error(), __LINE__); return 3; } } while (0)

static unsigned long long state = 88172645463325252ull;
static float uniform01(void)
{
    state ^= state << 13; state ^= state >> 7; state ^= state << 17;      /* xorshift64 */
    return (float)((state >> 40) * (1.0 / 16777216.0));
}

static double rel_l2(const float *a, const float *t, long n)
{
    double num = 0, den = 0;
    for (long i = 0; i < n; i++) { double d = (double)a[i] - (double)t[i]; num += d * d; den += (double)t[i] * (double)t[i]; }
    return sqrt(num / den);
}

int main(void)
{
    const int d = 3, c = 2;
    const long N = 60000, M = 25000;
    float *hX = malloc(sizeof(float) * N * d), *hY = malloc(sizeof(float) * M * d), *hb = malloc(sizeof(float) * N * c);
    float *hout = malloc(sizeof(float) * N * c), *href = malloc(sizeof(float) * N * c);
    for (long i = 0; i < N * d; i++) hX[i] = uniform01();
    for (long i = 0; i < M * d; i++) hY[i] = 0.2f + 0.6f * uniform01();
    for (long i = 0; i < N * c; i++) hb[i] = 2.f * uniform01() - 1.f;
    float *X, *Y, *b, *out, *ref;
    CHECK_HIP(hipMalloc((void **)&X, sizeof(float) * N * d));
    CHECK_HIP(hipMalloc((void **)&Y, sizeof(float) * M * d));
    CHECK_HIP(hipMalloc((void **)&b, sizeof(float) * N * c));
    CHECK_HIP(hipMalloc((void **)&out, sizeof(float) * N * c));
    CHECK_HIP(hipMalloc((void **)&ref, sizeof(float) * N * c));
    CHECK_HIP(hipMemcpy(X, hX, sizeof(float) * N * d, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(Y, hY, sizeof(float) * M * d, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(b, hb, sizeof(float) * N * c, hipMemcpyHostToDevice));
    f3m_params prm = {0.5f, 1000.f, 64, 0, 0.15f, 1000};
    printf("%s\n", f3m_version());

    /* one tree: X = Y */
    CHECK_F3M(f3m_kmvm_f32(d, X, N, NULL, 0, b, c, &prm, out, NULL));
    CHECK_F3M(f3m_exact_f32(d, X, N, X, N, b, c, prm.ls, ref, NULL));
    CHECK_HIP(hipMemcpy(hout, out, sizeof(float) * N * c, hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(href, ref, sizeof(float) * N * c, hipMemcpyDeviceToHost));
    const double e1 = rel_l2(hout, href, N * c);
    printf("kmvm X=Y: rel-L2 %.3e\n", e1);

    /* two trees through a plan: K(X,Y) v, then K(X,Y)^T u on the same plan */
    f3m_plan *plan = NULL;
    CHECK_F3M(f3m_plan_create(d, X, N, Y, M, &prm, NULL, &plan));
    printf("plan depth %d, symmetric %d\n", f3m_plan_depth(plan), f3m_plan_symmetric(plan));
    CHECK_F3M(f3m_plan_apply(plan, b, c, out, NULL));                    /* b read as (M, c) */
    CHECK_F3M(f3m_exact_f32(d, X, N, Y, M, b, c, prm.ls, ref, NULL));
    CHECK_HIP(hipMemcpy(hout, out, sizeof(float) * N * c, hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(href, ref, sizeof(float) * N * c, hipMemcpyDeviceToHost));
    const double e2 = rel_l2(hout, href, N * c);
    printf("plan K(X,Y) b: rel-L2 %.3e\n", e2);
    CHECK_F3M(f3m_plan_apply_transpose(plan, b, c, out, NULL));          /* b read as (N, c), result (M, c) */
    CHECK_F3M(f3m_exact_f32(d, Y, M, X, N, b, c, prm.ls, ref, NULL));
    CHECK_HIP(hipMemcpy(hout, out, sizeof(float) * M * c, hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(href, ref, sizeof(float) * M * c, hipMemcpyDeviceToHost));
    const double e3 = rel_l2(hout, href, M * c);
    printf("plan K(X,Y)^T u: rel-L2 %.3e\n", e3);
    CHECK_F3M(f3m_plan_destroy(plan));

    /* an error comes back as a code and a message */
    prm.ls = -1.f;
    if (f3m_kmvm_f32(d, X, N, NULL, 0, b, c, &prm, out, NULL) == 0) { printf("negative ls was accepted\n"); return 4; }
    printf("refused: %s\n", f3m_last_error());
    CHECK_F3M(f3m_release_cache());
    if (!(e1 < 1e-3 && e2 < 1e-3 && e3 < 1e-3)) { printf("FAILED\n"); return 1; }
    printf("OK\n");
    return 0;
}

// Host program of tests/test_dense16_plan.py: every plan t12_plan_dense16_heads makes over a sweep of shapes must
// describe a launch the kernel can run -- heads and tails inside their tensors, tails starting on a whole workgroup
// of the head size, all tails within one round -- and must not take more rounds than the plain launch.
#include <cstdint>
#include <cstdio>
#include <cstdlib>

#include "dense16_plan.h"

static uint64_t state = 0x9e3779b97f4a7c15ull;
static uint32_t rnd()
{
    state ^= state << 13;
    state ^= state >> 7;
    state ^= state << 17;
    return (uint32_t)(state >> 11);
}

int main(int argc, char** argv)
{
    const long cases = argc > 1 ? atol(argv[1]) : 200000;
    const int cu_choices[] = {1, 2, 7, 60, 64, 104, 228, 256, 304};
    long plans = 0, none = 0;
    for (long c = 0; c < cases; c++) {
        const int max_seg = 16;
        const int nseg = 1 + (int)(rnd() % 10);                       // more than max_seg / 2 must be refused
        const int rg = (rnd() & 1) ? 4 : 2;
        const int cus = cu_choices[rnd() % 9];
        int M[16], head[16];
        for (int i = 0; i < nseg; i++) {
            const uint32_t k = rnd() % 6;
            M[i] = k == 0 ? 1 + (int)(rnd() % 64) : (k == 1 ? 16 * (1 + (int)(rnd() % 2000)) : 1 + (int)(rnd() % 40000));
            head[i] = -12345;
        }
        const int rgb = t12_plan_dense16_heads(M, nseg, rg, cus, max_seg, head);
        if (rgb == 0) { none++; continue; }
        plans++;
        if (rgb < 1 || rgb >= rg || 2 * nseg > max_seg) { printf("bad rgb %d (rg %d, nseg %d)\n", rgb, rg, nseg); return 1; }
        long long head_wg = 0, tail_wg = 0, plain_wg = 0;
        for (int i = 0; i < nseg; i++) {
            if (head[i] < 0 || head[i] > M[i]) { printf("head %d outside tensor of %d rows\n", head[i], M[i]); return 1; }
            if (head[i] < M[i] && head[i] % (16 * rg)) { printf("tail starts inside a workgroup: %d of %d, rg %d\n", head[i], M[i], rg); return 1; }
            head_wg += (head[i] + 16 * rg - 1) / (16 * rg);
            tail_wg += (M[i] - head[i] + 16 * rgb - 1) / (16 * rgb);
            plain_wg += (M[i] + 16 * rg - 1) / (16 * rg);
        }
        if (tail_wg > cus) { printf("tails of %lld workgroups on %d CUs\n", tail_wg, cus); return 1; }
        const long long plain_rounds = (plain_wg + cus - 1) / cus, plan_rounds = (head_wg + cus - 1) / cus + (tail_wg > 0);
        if (plan_rounds > plain_rounds) { printf("plan takes %lld rounds, plain launch %lld\n", plan_rounds, plain_rounds); return 1; }
    }
    printf("ok: %ld plans checked, %ld launches left plain\n", plans, none);
    return plans > cases / 50 ? 0 : 2;                                 // (the sweep must reach the planner's main path)
}

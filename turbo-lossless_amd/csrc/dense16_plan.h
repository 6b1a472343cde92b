// Host-side planning of the small-batch sweep's launch with two sizes of workgroup (gemm.hip,
// gemm_dense16_mixed_kernel).  Plain integer arithmetic, no GPU types: compiled into the library and, by the tests,
// into a host program that checks every plan over a sweep of shapes.
#pragma once

// A launch of `nseg` tensors of M[i] rows, swept by workgroups of 16 * rg rows, one workgroup per CU at a time, on a chip
// of `cus` CUs.  When the last round of that launch would fill less than 7/8 of the chip, the plan cuts every tensor
// into a head of rows_head[i] rows (a multiple of 16 * rg, possibly 0), swept in whole rounds of 16 * rg-row
// workgroups, and a tail of M[i] - rows_head[i] rows swept by workgroups of 16 * rgb rows, rgb < rg, chosen so that all
// tails together are at most one round.  Returns rgb (1 .. rg - 1), or 0 when the plain launch is as good (one round
// or less, whole rounds, a nearly full last round, more than max_seg / 2 tensors, or no rgb that fits).
inline int t12_plan_dense16_heads(const int* M, int nseg, int rg, int cus, int max_seg, int* rows_head)
{
    if (nseg < 1 || rg < 2 || cus < 1 || 2 * nseg > max_seg) return 0;
    long long groups16 = 0, sets = 0;
    for (int i = 0; i < nseg; i++) {
        if (M[i] < 1) return 0;
        groups16 += (M[i] + 15) / 16;
        sets += (M[i] + 16 * rg - 1) / (16 * rg);
    }
    if (sets <= cus || sets % cus == 0 || (sets % cus) * 8 >= (long long)cus * 7) return 0;
    const long long full = (sets / cus) * cus;             // workgroups of the whole rounds
    long long rem_total = 0;
    int heads[64], rem[64];
    if (nseg > 64) return 0;
    for (int i = 0; i < nseg; i++) {
        const int gi = (M[i] + 15) / 16;
        int a = (int)(full * gi / groups16);               // this tensor's share of the whole rounds
        if ((long long)a * rg > gi) a = gi / rg;
        heads[i] = a;
        rem[i] = gi - a * rg;
        rem_total += rem[i];
    }
    int rgb = (int)((rem_total + cus - 1) / cus);
    for (; rgb >= 1 && rgb < rg; rgb++) {
        long long b = 0;
        for (int i = 0; i < nseg; i++) b += (rem[i] + rgb - 1) / rgb;
        if (b <= cus) break;
    }
    if (rgb < 1 || rgb >= rg) return 0;
    for (int i = 0; i < nseg; i++) {
        const long long r = 16LL * rg * heads[i];
        rows_head[i] = (int)(r < M[i] ? r : M[i]);
    }
    return rgb;
}

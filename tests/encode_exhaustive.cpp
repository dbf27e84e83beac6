// Host-side exhaustive check of lpmm_encode.hpp: for every fp32 bit pattern that is not a NaN,
// the table-driven first-moment code and the closed-form second-moment code must equal the
// reference search (upper bound + midpoint test) restated here.
// Build: g++ -O2 -fopenmp -ffp-contract=off -I<csrc> encode_exhaustive.cpp
#include <cstdint>
#include <cstdio>
#include <cstring>

#include "lpmm_encode.hpp"

using namespace lpmm;

static int ref_search(const float *q, float x)
{
    int lo = 0, hi = 16;
    if (x <= q[0]) return 0;
    if (q[15] <= x) return 15;
    while (lo < hi) {
        int mi = (lo + hi) >> 1;
        if (q[mi] <= x) lo = mi + 1; else hi = mi;
    }
    float mid = (q[lo - 1] + q[lo]) * 0.5f;
    return (mid < x) ? lo : lo - 1;
}

int main()
{
    float qm[16], qv[16];
    memcpy(qm, kStdQmapMBits, sizeof qm);
    memcpy(qv, kStdQmapVBits, sizeof qv);
    long long bad_m = 0, bad_v = 0, checked = 0;
#pragma omp parallel for reduction(+ : bad_m, bad_v, checked) schedule(static)
    for (long long i = 0; i < (1LL << 32); ++i) {
        const uint32_t xb = (uint32_t)i;
        if ((xb & 0x7fffffffu) > 0x7f800000u) continue;  // NaN
        float x;
        memcpy(&x, &xb, 4);
        // the table is indexed by the bucket byte (the 8-bit float conversion, restated on the host)
        const uint32_t bucket = enc_m_bucket_host(x);
        if (bucket >= (uint32_t)kEncEntries) { ++bad_m; continue; }
        const uint32_t *e = kEncTableM[enc_m_stored_index(bucket)];
        if ((int)enc_m_pick(x, e[0], e[1], e[2]) != ref_search(qm, x)) ++bad_m;
        if ((int)enc_v_linear(x) != ref_search(qv, x)) ++bad_v;
        ++checked;
    }
    printf("checked %lld bad_m %lld bad_v %lld\n", checked, bad_m, bad_v);
    return (bad_m || bad_v) ? 1 : 0;
}

// The fused lm_head -> logprob kernel for calls of few rows (included by ka_lmhead.hip, which defines the tiling
// constants, the split plan, the partials and the folds that this file uses).
//
// With at most a few hundred rows the operator streams W once and is bound by memory, not by the matrix pipes: what
// matters is how many bytes a CU has in flight.  This kernel keeps the work decomposition of lmhead_partials - units
// of a vocabulary split as work items, 256-row vocabulary tiles, slabs of 64 along the hidden dimension, the same
// MFMA operand layout, the same order of every floating-point operation that touches a row's result, so results are
// the same bit for bit - but its workgroup covers 64 * TN tokens instead of 256 (TN = 1 or 2 blocks of 32 tokens per
// wavefront): the hidden slab shrinks from 32 KB to 8 * TN KB, three stages fit in LDS instead of two, and the copies
// of a slab are requested two slabs ahead.  One barrier per slab; no instruction scheduling by hand (the MFMAs are a
// quarter or a half of the large kernel's and never the bound).
#ifndef KA_LMHEAD_NARROW_H
#define KA_LMHEAD_NARROW_H

namespace ka {
namespace {

constexpr int LN_STAGES = 3;
template <int TN> constexpr int ln_stage_bytes() { return (LM_BM + 64 * TN) * LM_BK * 2; }
template <int TN> constexpr int ln_lds_bytes() { return LN_STAGES * ln_stage_bytes<TN>() + LM_XCH_BYTES; }

template <int TN, bool ENTROPY>
__global__ __launch_bounds__(LM_THREADS, 1) void lmhead_partials_narrow(
    const uint16_t *__restrict__ hidden, const uint16_t *__restrict__ weight, const int64_t *__restrict__ ids,
    Partial *__restrict__ partials, int n_rows, int hdim, int vocab, int n_token_blocks, SplitPlan plan, int n_virtual) {
    extern __shared__ __attribute__((aligned(16))) uint16_t lds[];  // [stage][W slab 256 x 64 | hidden slab 64 TN x 64], then the exchange area
    constexpr int BN = 64 * TN;                    // tokens per workgroup
    constexpr int STAGE = ln_stage_bytes<TN>();    // bytes
    constexpr int HCOPIES = 2 * TN;                // hidden copies per slab (32 rows each)
    constexpr int CPS = 8 + HCOPIES;               // copies per slab and wavefront
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wave_m = wave >> 1, wave_n = wave & 1, l32 = lane & 31, lhalf = lane >> 5;
    const ItemOrder order(n_token_blocks, plan, 1);  // items are (token block, unit) pairs
    const int stride = gridDim.x, nk = hdim / LM_BK;
    int v = blockIdx.x, tb, u;
    if (!lm_decode(v, order, tb, u)) v = lm_next_item(v, stride, n_virtual, order);
    if (v >= n_virtual) return;

    // ---- copies (same lane mapping as lmhead_partials: instruction j of wavefront w covers rows (4 j + w) * 8 .. + 7) ----
    const int cp_row = wave * 8 + (lane >> 3);
    const uint32_t row_bytes = uint32_t(hdim) * 2u;
    const char *const wbytes = reinterpret_cast<const char *>(weight);
    const char *const hbytes = reinterpret_cast<const char *>(hidden);
    const int wave_lds = __builtin_amdgcn_readfirstlane(wave) * 1024;  // bytes: 8 rows of 128
    struct Cursor { int v, tb, vt, vt_end, kt; } cur;
    cur.v = v; cur.tb = tb; cur.vt = order.col_begin(u); cur.vt_end = order.col_begin(u + 1); cur.kt = 0;
    auto issue = [&](const Cursor &c, int stage) {
        const uint32_t kb = uint32_t(c.kt) * (LM_BK * 2);
        char *const base = reinterpret_cast<char *>(lds) + stage * STAGE + wave_lds;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int row = cp_row + 32 * j;
            const uint32_t off = uint32_t(min(c.vt * LM_BM + row, vocab - 1)) * row_bytes + uint32_t(((lane & 7) ^ swz(row)) * 16);
            __builtin_amdgcn_global_load_lds(wbytes + kb + off, (lds_void *)(base + j * 4096), 16, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < HCOPIES; ++j) {
            const int row = cp_row + 32 * j;
            const uint32_t off = uint32_t(min(c.tb * BN + row, n_rows - 1)) * row_bytes + uint32_t(((lane & 7) ^ swz(row)) * 16);
            __builtin_amdgcn_global_load_lds(hbytes + kb + off, (lds_void *)(base + LM_BM * LM_BK * 2 + j * 4096), 16, 0, 0);
        }
    };
    // the slab behind c (past the last slab of the workgroup's last item the cursor stays: redundant copies keep
    // the count of copies per slab, which the waits rely on, constant)
    auto advance = [&](Cursor &c) {
        if (c.kt + 1 < nk) { ++c.kt; return; }
        if (c.vt + 1 < c.vt_end) { ++c.vt; c.kt = 0; return; }
        const int nv = lm_next_item(c.v, stride, n_virtual, order);
        if (nv >= n_virtual) return;
        int tb2, u2;
        lm_decode(nv, order, tb2, u2);
        c.v = nv; c.tb = tb2; c.vt = order.col_begin(u2); c.vt_end = order.col_begin(u2 + 1); c.kt = 0;
    };

    // ---- fragment addresses (as in lmhead_partials) ----
    typedef __attribute__((address_space(3))) const unsigned char lds_cbyte;
    typedef __attribute__((address_space(3))) const bf16x8 lds_frag;
    lds_cbyte *const lds3 = (lds_cbyte *)lds;
    int fa_off[4], fb_off[4];
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
        const int chunk = ((kk * 2 + lhalf) ^ swz(l32)) << 4;
        fa_off[kk] = (wave_m * 128 + l32) * (LM_BK * 2) + chunk;
        fb_off[kk] = (LM_BM + wave_n * (32 * TN) + l32) * (LM_BK * 2) + chunk;
    }
    float *const xch = reinterpret_cast<float *>(reinterpret_cast<char *>(lds) + LN_STAGES * STAGE);  // [wave_n][tn][32][4]
    const bool folder = wave_m == 0 && lhalf == 0;

    issue(cur, 0);
    advance(cur);
    issue(cur, 1);
    advance(cur);
    int stage = 0;  // stage of the slab being multiplied

    float m_run[TN], ml2_run[TN], s_run[TN], xt[TN], a_run[TN];
    int target[TN];
    for (;;) {  // items of this workgroup
    lm_decode(v, order, tb, u);
    const int tok0 = tb * BN;
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
        const int n = tok0 + wave_n * (32 * TN) + tn * 32 + l32;
        int64_t id = -1;
        if (n < n_rows) id = ids[n];
        target[tn] = (id >= 0 && id < vocab) ? int(id) : -1;
        m_run[tn] = kFloor;
        ml2_run[tn] = kFloor * kLog2e;
        s_run[tn] = 0.0f;
        a_run[tn] = 0.0f;
        xt[tn] = -__builtin_inff();
    }
    const int vt_begin = order.col_begin(u), vt_end = order.col_begin(u + 1);
    for (int vt = vt_begin; vt < vt_end; ++vt) {
        f32x16 acc[4][TN];
#pragma unroll
        for (int tm = 0; tm < 4; ++tm)
#pragma unroll
            for (int tn = 0; tn < TN; ++tn)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[tm][tn][r] = 0.0f;
        for (int kt = 0; kt < nk; ++kt) {
            // The slab to multiply has landed once at most the copies of the slab behind it are outstanding (copies
            // complete in order); behind the barrier every wavefront has also finished with the slab before it, whose
            // stage takes the copies of the slab two ahead.
            asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(CPS) : "memory");
            issue(cur, stage == 0 ? 2 : stage - 1);
            advance(cur);
            lds_cbyte *const sbase = lds3 + stage * STAGE;
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) {
                bf16x8 fa[4], fb[TN];
#pragma unroll
                for (int t = 0; t < 4; ++t) fa[t] = *(lds_frag *)(sbase + fa_off[kk] + t * (32 * LM_BK * 2));
#pragma unroll
                for (int t = 0; t < TN; ++t) fb[t] = *(lds_frag *)(sbase + fb_off[kk] + t * (32 * LM_BK * 2));
#pragma unroll
                for (int tm = 0; tm < 4; ++tm)
#pragma unroll
                    for (int tn = 0; tn < TN; ++tn)
                        acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[tm], fb[tn], acc[tm][tn], 0, 0, 0);
            }
            stage = stage == 2 ? 0 : stage + 1;
        }

        // ---- the logits of this vocabulary tile are complete: the same fold as in lmhead_partials ----
        const int vrow0 = vt * LM_BM + wave_m * 128 + lhalf * 4;
        const int limit = vocab - vrow0;
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
#pragma clang fp contract(off)
            const int d = target[tn] - (vt * LM_BM + wave_m * 128);
            const bool mine = d >= 0 && d < 128 && ((d >> 2) & 1) == lhalf;
            const int want = mine ? (((d >> 5) << 4) | ((d & 31) >> 3 << 2) | (d & 3)) : -1;  // tm*16 + r
            float mn = m_run[tn];
            float part[4], parta[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            if (limit >= 128 && !__any(mine)) {
#pragma unroll
                for (int tm = 0; tm < 4; ++tm)
#pragma unroll
                    for (int r = 0; r < 16; ++r) mn = fmaxf(mn, acc[tm][tn][r]);
                const float ml2f = mn * kLog2e;
#pragma unroll
                for (int tm = 0; tm < 4; ++tm) {
                    float e[16];
#pragma unroll
                    for (int r = 0; r < 16; ++r) e[r] = fast_exp2(fmaf(acc[tm][tn][r], kLog2e, -ml2f));
                    if constexpr (ENTROPY) {
                        float xe[16];
#pragma unroll
                        for (int r = 0; r < 16; ++r) xe[r] = acc[tm][tn][r] * e[r];
#pragma unroll
                        for (int step = 1; step < 16; step <<= 1)
#pragma unroll
                            for (int r = 0; r + step < 16; r += 2 * step) xe[r] += xe[r + step];
                        parta[tm] = xe[0];
                    }
#pragma unroll
                    for (int step = 1; step < 16; step <<= 1)
#pragma unroll
                        for (int r = 0; r + step < 16; r += 2 * step) e[r] += e[r + step];
                    part[tm] = e[0];
                }
            } else {
#pragma unroll
                for (int tm = 0; tm < 4; ++tm)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const float x = (tm * 32 + (r >> 2) * 8 + (r & 3) < limit) ? acc[tm][tn][r] : -__builtin_inff();
                        mn = fmaxf(mn, x);
                        if (want == tm * 16 + r) xt[tn] = x;
                    }
                const float ml2s = mn * kLog2e;
#pragma unroll
                for (int tm = 0; tm < 4; ++tm) {
                    float e[16];
                    float xe[16];
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const float x = (tm * 32 + (r >> 2) * 8 + (r & 3) < limit) ? acc[tm][tn][r] : -__builtin_inff();
                        e[r] = fast_exp2(fmaf(x, kLog2e, -ml2s));
                        if constexpr (ENTROPY) xe[r] = e[r] == 0.0f ? 0.0f : x * e[r];
                    }
                    if constexpr (ENTROPY) {
#pragma unroll
                        for (int step = 1; step < 16; step <<= 1)
#pragma unroll
                            for (int r = 0; r + step < 16; r += 2 * step) xe[r] += xe[r + step];
                        parta[tm] = xe[0];
                    }
#pragma unroll
                    for (int step = 1; step < 16; step <<= 1)
#pragma unroll
                        for (int r = 0; r + step < 16; r += 2 * step) e[r] += e[r + step];
                    part[tm] = e[0];
                }
            }
            const float ml2n = mn * kLog2e;
            const float rescale = fast_exp2(ml2_run[tn] - ml2n);
            s_run[tn] = fmaf(s_run[tn], rescale, (part[0] + part[1]) + (part[2] + part[3]));
            if constexpr (ENTROPY) a_run[tn] = fmaf(a_run[tn], rescale, (parta[0] + parta[1]) + (parta[2] + parta[3]));
            m_run[tn] = mn;
            ml2_run[tn] = ml2n;
        }
    }

    // ---- end of the unit: the two lane halves, then the two vocabulary halves of the tile (as in lmhead_partials) ----
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
        const float om = __shfl_xor(m_run[tn], 32, kWave);
        const float os = __shfl_xor(s_run[tn], 32, kWave);
        const float ox = __shfl_xor(xt[tn], 32, kWave);
        const float mm = fmaxf(m_run[tn], om);
        const float lo_s = lhalf == 0 ? s_run[tn] : os, lo_m = lhalf == 0 ? m_run[tn] : om;
        const float hi_s = lhalf == 0 ? os : s_run[tn], hi_m = lhalf == 0 ? om : m_run[tn];
        const float f_lo = fast_exp2((lo_m - mm) * kLog2e), f_hi = fast_exp2((hi_m - mm) * kLog2e);
        s_run[tn] = lo_s * f_lo + hi_s * f_hi;
        if constexpr (ENTROPY) {
            const float oa = __shfl_xor(a_run[tn], 32, kWave);
            const float lo_a = lhalf == 0 ? a_run[tn] : oa, hi_a = lhalf == 0 ? oa : a_run[tn];
            a_run[tn] = lo_a * f_lo + hi_a * f_hi;
        }
        m_run[tn] = mm;
        xt[tn] = fmaxf(xt[tn], ox);
    }
    if (wave_m == 1 && lhalf == 0) {
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
            float *p = xch + ((wave_n * 4 + tn) * 32 + l32) * 4;
            p[0] = m_run[tn];
            p[1] = s_run[tn];
            p[2] = xt[tn];
            if constexpr (ENTROPY) p[3] = a_run[tn];
        }
    }
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0) only: the slab copies in flight are not waited for
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (folder) {
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
            const float *p = xch + ((wave_n * 4 + tn) * 32 + l32) * 4;
            const float om = p[0], os = p[1], ox = p[2];
            const float mm = fmaxf(m_run[tn], om);
            const float f_own = fast_exp2((m_run[tn] - mm) * kLog2e), f_other = fast_exp2((om - mm) * kLog2e);
            const float s = s_run[tn] * f_own + os * f_other;
            float a = 0.0f;
            if constexpr (ENTROPY) a = a_run[tn] * f_own + p[3] * f_other;
            const float x = fmaxf(xt[tn], ox);
            const int n = tok0 + wave_n * (32 * TN) + tn * 32 + l32;
            if (n < n_rows) {
                Partial out;
                out.m = mm;
                out.s = s;
                out.xt = x;
                out.pad = a;
                partials[size_t(u) * n_rows + n] = out;
            }
        }
    }
    v = lm_next_item(v, stride, n_virtual, order);
    if (v >= n_virtual) break;
    }  // items
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): the trailing (redundant) slab copies still write LDS
}

}  // namespace
}  // namespace ka

#endif  // KA_LMHEAD_NARROW_H

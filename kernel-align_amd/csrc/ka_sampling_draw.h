// The draw of the radix path for 16-byte aligned rows of any dtype: the first survivor, in index order, whose
// inclusive integer mass exceeds floor(u * Z).
#ifndef KA_SAMPLING_DRAW_H
#define KA_SAMPLING_DRAW_H

#include "ka_sampling_common.h"
#include "ka_sampling_dense.h"

namespace ka {
namespace {

// Survivors are the entries with key > kcut and, of the entries equal to kcut, the first r_cut in index order
// (all of them when r_cut is 0xffffffff).  Every wavefront sums the survivors of a contiguous sixteenth of the
// row (one evaluation of the mass polynomial per survivor), the sixteenth that holds floor(u * Z) is then
// searched by all wavefronts, one 64-vector step each, and the wavefront whose step holds it finds the lane and
// the entry: about 1 + 1/16 evaluations per entry, three barriers, no block-wide scan per tile of the row.
// Returns Z (the total mass of the survivors) through *z_out.
template <typename T>
__device__ __forceinline__ void draw_by_shares(DenseScalars &ds, const typename T::raw_t *rp, int vocab, float temp,
                                               bool has_t, uint32_t kmax, float vmax, uint32_t kcut, uint32_t r_cut,
                                               float u, int64_t *out_slot, float *lp_slot) {
    constexpr int EPV = T::kPerVec;
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1), wave = tid / kWave;
    const bool track = r_cut != 0xffffffffu;
    auto weight = [&](uint32_t key) -> uint64_t { return weight_fix(key == kmax ? 0.0f : value_of<T>(key) - vmax); };
    const uint64_t w_tie = track ? weight(kcut) : 0ull;
    // mass of the full survivors of one vector and its number of tie-group entries (rolled: the polynomial is long)
    auto vector_sums = [&](const uint4 &q, uint64_t &m, uint32_t &t) {
        const typename T::raw_t *e = reinterpret_cast<const typename T::raw_t *>(&q);
#pragma unroll 2
        for (int j = 0; j < EPV; ++j) {
            const uint32_t key = elem_key<T>(e[j], temp, has_t);
            if (key > kcut || (key == kcut && !track)) m += weight(key);
            else if (key == kcut) ++t;
        }
    };
    const int nvec = vocab / EPV;
    const int vpw = (nvec + S_WAVES - 1) / S_WAVES;  // vectors per wavefront
    const uint4 *const vrow = reinterpret_cast<const uint4 *>(rp);
    // the ragged tail of the row: fewer than EPV entries after the last vector, one per lane of wavefront 0
    const int tail_index = nvec * EPV + tid;
    const bool has_tail = tail_index < vocab;
    const uint32_t tail_key = has_tail ? elem_key<T>(rp[tail_index], temp, has_t) : 0u;
    const bool tail_tie = has_tail && track && tail_key == kcut;
    const uint64_t tail_mass = (has_tail && !tail_tie && tail_key >= kcut) ? weight(tail_key) : 0ull;

    // a. per wavefront: its share of the row
    {
        const int v0 = wave * vpw;
        const int n_here = nvec - v0 < vpw ? (nvec - v0 > 0 ? nvec - v0 : 0) : vpw;
        uint64_t m = 0;
        uint32_t t = 0;
#pragma unroll 1
        for (int i0 = 0; i0 < n_here; i0 += 4 * kWave) {
            uint4 q[4];
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const int idx = i0 + s * kWave + lane;
                q[s] = idx < n_here ? vrow[v0 + idx] : make_uint4(0, 0, 0, 0);
            }
#pragma unroll 1
            for (int s = 0; s < 4; ++s)
                if (i0 + s * kWave + lane < n_here) vector_sums(q[s], m, t);
        }
        m = wave_sum_u64(m);
        t = wave_sum_u32(t);
        uint64_t mt = tail_mass;
        uint32_t tt = tail_tie ? 1u : 0u;
        if (wave == 0) {
            mt = wave_sum_u64(mt);
            tt = wave_sum_u32(tt);
        }
        if (lane == 0) {
            ds.seg_mass[wave] = m;
            ds.seg_ties[wave] = t;
            if (wave == 0) {
                ds.seg_mass[S_WAVES] = mt;
                ds.seg_ties[S_WAVES] = tt;
                ds.hit = -1;
            }
        }
    }
    __syncthreads();
    // b. the segment (a wavefront's share, or the tail) that holds floor(u * Z)
    uint64_t z = 0;
    {
        uint32_t seen = 0;
#pragma unroll
        for (int g = 0; g <= S_WAVES; ++g) {
            const uint32_t t = ds.seg_ties[g];
            const uint32_t room = seen < r_cut ? r_cut - seen : 0u;
            z += ds.seg_mass[g] + uint64_t(t < room ? t : room) * w_tie;
            seen += t;
        }
    }
    const uint64_t tau = floor_scale(u, z);
    uint64_t acc = 0;          // mass before the segment
    uint32_t ties_before = 0;  // tie-group entries before the segment
    int seg = -1;
    {
        uint32_t seen = 0;
#pragma unroll
        for (int g = 0; g <= S_WAVES; ++g) {
            const uint32_t t = ds.seg_ties[g];
            const uint32_t room = seen < r_cut ? r_cut - seen : 0u;
            const uint64_t m = ds.seg_mass[g] + uint64_t(t < room ? t : room) * w_tie;
            if (seg < 0 && tau < acc + m) { seg = g; ties_before = seen; }
            if (seg < 0) acc += m;
            seen += t;
        }
    }
    // c. inside the segment, in rounds of S_WAVES steps of 64 vectors
    if (seg >= 0 && seg < S_WAVES) {  // the same for the whole block
        const int sv0 = seg * vpw;
        const int n_seg = nvec - sv0 < vpw ? nvec - sv0 : vpw;
        const int n_steps = (n_seg + kWave - 1) / kWave;
        uint64_t cum = acc;
        uint32_t rank = ties_before;
        for (int st0 = 0; st0 < n_steps; st0 += S_WAVES) {  // block-uniform trip count and exit
            const int idx = (st0 + wave) * kWave + lane;
            const bool valid = idx < n_seg;
            const uint4 q = valid ? vrow[sv0 + idx] : make_uint4(0, 0, 0, 0);
            uint64_t m = 0;
            uint32_t t = 0;
            if (valid) vector_sums(q, m, t);
            const uint64_t ms = wave_sum_u64(m);
            const uint32_t ts = wave_sum_u32(t);
            if (lane == 0) {
                ds.wave_u64[wave] = ms;
                ds.wave_u32[wave] = ts;
            }
            __syncthreads();
            uint64_t hcum = 0;
            uint32_t hrank = 0;
            int hstep = -1;
#pragma unroll
            for (int st = 0; st < S_WAVES; ++st) {
                if (st0 + st < n_steps) {
                    const uint32_t st_ties = ds.wave_u32[st];
                    const uint32_t room = rank < r_cut ? r_cut - rank : 0u;
                    const uint64_t total = ds.wave_u64[st] + uint64_t(st_ties < room ? st_ties : room) * w_tie;
                    if (hstep < 0 && tau < cum + total) {
                        hstep = st;
                        hcum = cum;
                        hrank = rank;
                    }
                    cum += total;
                    rank += st_ties;
                }
            }
            if (hstep >= 0) {
                if (wave == hstep) {
                    // lanes of that step in order: tie ranks first, then masses
                    const uint32_t rk0 = hrank + wave_excl_scan<uint32_t>(t);
                    const uint32_t room = rk0 < r_cut ? r_cut - rk0 : 0u;
                    const uint64_t lm = m + uint64_t(t < room ? t : room) * w_tie;
                    const uint64_t before = hcum + wave_excl_scan<uint64_t>(lm);
                    if (before <= tau && tau < before + lm) {
                        const typename T::raw_t *e = reinterpret_cast<const typename T::raw_t *>(&q);
                        uint64_t c2 = before;
                        uint32_t r2 = rk0;
#pragma unroll 1
                        for (int j = 0; j < EPV; ++j) {
                            const uint32_t key = elem_key<T>(e[j], temp, has_t);
                            uint64_t wj = 0;
                            if (key > kcut || (key == kcut && !track)) wj = weight(key);
                            else if (key == kcut) wj = (r2++ < r_cut) ? w_tie : 0ull;
                            c2 += wj;
                            if (c2 > tau) {
                                ds.hit = int64_t(sv0 + idx) * EPV + j;
                                ds.pick_w = wj;
                                break;
                            }
                        }
                    }
                }
                break;
            }
            __syncthreads();  // the per-step totals are overwritten by the next round
        }
    } else if (seg == S_WAVES && wave == 0) {
        const uint32_t rk = ties_before + wave_excl_scan<uint32_t>(tail_tie ? 1u : 0u);
        const uint64_t wt = tail_tie ? (rk < r_cut ? w_tie : 0ull) : tail_mass;
        const uint64_t before = acc + wave_excl_scan<uint64_t>(wt);
        if (before <= tau && tau < before + wt) {
            ds.hit = tail_index;
            ds.pick_w = wt;
        }
    }
    __syncthreads();
    if (tid == 0) {
        *out_slot = ds.hit;
        if (lp_slot != nullptr) *lp_slot = ds.hit >= 0 ? log_ratio(ds.pick_w, z) : __builtin_nanf("");
    }
}

}  // namespace
}  // namespace ka

#endif  // KA_SAMPLING_DRAW_H

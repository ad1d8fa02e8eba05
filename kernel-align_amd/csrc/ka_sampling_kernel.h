// The sampling kernel itself: one workgroup per row, all routes (included by the two builds of the kernel: 1024 threads per
// row, and 512 for the top-k route of large batches).
#ifndef KA_SAMPLING_KERNEL_H
#define KA_SAMPLING_KERNEL_H

#include "ka_sampling_common.h"
#include "ka_sampling_dense.h"
#include "ka_sampling_topk.h"
#include "ka_sampling_draw.h"

namespace ka {

// Per-launch parameters.  Each of the three filter parameters is either one value for the whole batch or,
// when its *_rows pointer is set, one value per row; a row value that is not valid switches that filter
// off (temperature <= 0 or NaN -> 1, top_k < 0 -> off, top_p outside (0, 1] -> off).
struct SampleParams {
    float temperature;
    int top_k;
    float top_p;
    const float *temperature_rows;
    const int32_t *top_k_rows;
    const float *top_p_rows;
    const float *uniforms;
    int64_t *out_ids;
    float *out_logprob;  // optional: log of the sampled entry's probability under the filtered distribution
    float *out_policy;   // optional: its log-probability under the unfiltered softmax of the raw logits
};

// Launch of the 512-thread build of sample_rows<T, false> (defined in ka_sampling_half.hip); the row is 16-byte aligned
// and holds at most 32 * 512 vectors (16-bit dtypes) or 4 * 32 * 512 (fp32).
hipError_t launch_sample_rows_half(int dtype, const void *logits, int64_t batch, int vocab, int64_t row_stride,
                                   const SampleParams &prm, int path_bits, hipStream_t stream);

namespace {

// ---------------------------------------------------------------------------
// The kernel
// ---------------------------------------------------------------------------
// DENSE = launched with DENSE_LDS_BYTES of dynamic LDS: the dense-histogram path is available, and the state
// of the other paths sits at the start of the same memory (the paths never run at the same time).
template <bool DENSE> __device__ __forceinline__ unsigned char *lds_base() {
    if constexpr (DENSE) {
        extern __shared__ __attribute__((aligned(16))) unsigned char dyn_lds[];
        return dyn_lds;
    } else {
        __shared__ Shared static_lds;
        return reinterpret_cast<unsigned char *>(&static_lds);
    }
}

// One row.  Returns 1 when the row's id (and filtered log-probability) is written or on its way (on some routes one
// wavefront still finishes while the others return), 2 when the same holds for the policy log-probability.
template <typename T, bool DENSE>
__device__ __forceinline__ int sample_one_row(const typename T::raw_t *__restrict__ logits, int vocab, int64_t row_stride,
                                              const SampleParams &prm, int vec, int no_fast, PolicyLse &lse) {
    constexpr int EPV = T::kPerVec;
    constexpr int LEVELS = Round<T>::kLevels;
    // For fp32 rows the second variant is the radix path alone, with the draw done by shares of the row; the host
    // launches it for the filter combinations that the top-k fast path does not serve.  (Kept apart because the
    // register allocation of the fast path suffers when the code behind it grows.)
    constexpr bool RADIX_ONLY = DENSE && T::kBytes == 4;
    unsigned char *const lds = lds_base<DENSE && T::kBytes == 2>();
    Shared &sh = *reinterpret_cast<Shared *>(lds);
    const int tid = threadIdx.x;
    const int64_t row = blockIdx.x;
    const typename T::raw_t *rp = logits + row * row_stride;
    float temp = prm.temperature;
    int top_k = prm.top_k;
    float top_p = prm.top_p;
    if (prm.temperature_rows != nullptr) { temp = prm.temperature_rows[row]; if (!(temp > 0.0f)) temp = 1.0f; }
    if (prm.top_k_rows != nullptr) { top_k = prm.top_k_rows[row]; if (top_k < 0) top_k = 0; }
    if (prm.top_p_rows != nullptr) { top_p = prm.top_p_rows[row]; if (!(top_p > 0.0f && top_p <= 1.0f)) top_p = 1.0f; }
    const float *__restrict__ uniforms = prm.uniforms;
    int64_t *out = prm.out_ids;  // (not restrict: the kernel reads the id back through prm.out_ids for the policy log-probability)
    float *lp_slot = prm.out_logprob != nullptr ? prm.out_logprob + row : nullptr;
    const bool has_t = temp != 1.0f;
    const bool use_k = top_k > 0 && top_k < vocab;
    const bool use_p = top_p < 1.0f;

    KA_STAMP(0);
    float u = uniforms[row];
    if (!(u >= 0.0f)) u = 0.0f;
    if (u >= 1.0f) u = __uint_as_float(0x3f7fffffu);

    // no_fast: bit 0 = take the general radix path, bit 1 = keep the top-k route block-wide (KA_SAMPLE_FLAG_*)
    if (!RADIX_ONLY && use_k && top_k <= S_THREADS && !(no_fast & 1)) {
        if constexpr (!RADIX_ONLY) {
            const int done = fast_topk<T>(sh, rp, vocab, vec, temp, has_t, top_k, use_p, top_p, u, out + row, lp_slot,
                                          (no_fast & 2) != 0, prm.out_policy != nullptr ? prm.out_policy + row : nullptr, lse);
            if (done) return done;
        }
        __syncthreads();
    } else if (!(no_fast & 1)) {
        if constexpr (DENSE && T::kBytes == 2) {
            bool done;
            if (!use_k && !use_p)
                done = has_t ? dense_stream<T, true, true>(lds, rp, vocab, vec, temp, false, 0, false, 1.0f, u, out + row, lp_slot)
                             : dense_stream<T, false, true>(lds, rp, vocab, vec, temp, false, 0, false, 1.0f, u, out + row, lp_slot);
            else
                done = has_t ? dense_stream<T, true, false>(lds, rp, vocab, vec, temp, use_k, top_k, use_p, top_p, u,
                                                            out + row, lp_slot)
                             : dense_stream<T, false, false>(lds, rp, vocab, vec, temp, use_k, top_k, use_p, top_p, u,
                                                             out + row, lp_slot);
            if (done) return 1;
            __syncthreads();
        }
        if constexpr (!DENSE && T::kBytes == 2 && S_THREADS == 1024) {
            if (!use_k && !use_p) {  // launched without the histogram's LDS: fp16, whose rows hold too many distinct values
                if (nofilter_resident<T>(sh.ds, rp, vocab, vec, temp, has_t, u, out + row, lp_slot)) return 1;
                __syncthreads();
            }
        }
    }

    // ---- pass 0: row maximum and the level-0 count histogram --------------------------
    clear_hist(sh);
    __syncthreads();
    uint32_t kmax = 0;
    for_each_key<T>(rp, vocab, vec, temp, has_t, [&](int, uint32_t key) {
        kmax = key > kmax ? key : kmax;
        if (use_k) atomicAdd(&sh.h.cnt[key >> 21], 1u);
    });
    kmax = block_max_u32(kmax, sh);  // barriers inside also publish the histogram
    const float vmax = value_of<T>(kmax);

    // ---- top-k: MSB-first descent to the k-th largest key --------------------------------
    uint32_t kstar = 0;      // keep key >= kstar
    uint32_t n_eq_kstar = 0; // entries equal to kstar (only meaningful with use_k)
    if (use_k) {
        uint32_t rank = uint32_t(top_k);  // 1-based rank inside the current prefix
        uint32_t prefix = 0;
        for (int level = 0; level < LEVELS; ++level) {
            const int shift = level_shift<T>(level), bits = level_bits<T>(level);
            const uint32_t nb = 1u << bits;
            if (level > 0) {
                clear_hist(sh);
                __syncthreads();
                const int pshift = level_shift<T>(level - 1);
                for_each_key<T>(rp, vocab, vec, temp, has_t, [&](int, uint32_t key) {
                    if ((key >> pshift) == prefix) atomicAdd(&sh.h.cnt[(key >> shift) & (nb - 1)], 1u);
                });
                __syncthreads();
            }
            uint32_t above;
            const uint32_t digit = select_count_bin(sh, nb, rank, &above, &n_eq_kstar);
            prefix = (prefix << bits) | digit;
            rank -= above;
        }
        kstar = prefix << level_shift<T>(LEVELS - 1);
    }

    // ---- masses of the survivors of top-k: total, and level-0 histogram for top-p ---------
    // (the draw by shares finds the total itself: without top-p this pass is not needed)
    uint64_t z_topk = 0;
    if (!(RADIX_ONLY && vec && !use_p)) {
        clear_hist(sh);
        __syncthreads();
        uint64_t zpart = 0;
        for_each_key<T>(rp, vocab, vec, temp, has_t, [&](int, uint32_t key) {
            if (key >= kstar) {
                const float y = value_of<T>(key);
                const uint64_t w = weight_fix(key == kmax ? 0.0f : y - vmax);
                zpart += w;
                if (use_p) {
                    atomicAdd(reinterpret_cast<unsigned long long *>(&sh.h.mass[key >> 21]), (unsigned long long)w);
                    atomicAdd(&sh.h.cnt[key >> 21], 1u);
                }
            }
        });
        block_excl_scan<uint64_t>(zpart, sh.wave_u64, &z_topk);
        __syncthreads();
    }

    // ---- top-p: descent to the lowest key whose first entry is still kept ------------------
    uint32_t kcut = kstar;            // survivors: key > kcut, or key == kcut with tie rank < r_cut
    uint32_t r_cut = 0xffffffffu;
    uint64_t z_kept = z_topk;
    if (use_p) {
        const uint64_t theta = floor_scale(top_p, z_topk);
        uint64_t before = 0;          // mass of the keys above the current prefix
        uint32_t prefix = 0;
        uint32_t n_cut = 0;
        uint64_t m_cut = 0;
        for (int level = 0; level < LEVELS; ++level) {
            const int shift = level_shift<T>(level), bits = level_bits<T>(level);
            const uint32_t nb = 1u << bits;
            if (level > 0) {
                clear_hist(sh);
                __syncthreads();
                const int pshift = level_shift<T>(level - 1);
                for_each_key<T>(rp, vocab, vec, temp, has_t, [&](int, uint32_t key) {
                    if (key >= kstar && (key >> pshift) == prefix) {
                        const float y = value_of<T>(key);
                        const uint64_t w = weight_fix(key == kmax ? 0.0f : y - vmax);
                        const uint32_t d = (key >> shift) & (nb - 1);
                        atomicAdd(reinterpret_cast<unsigned long long *>(&sh.h.mass[d]), (unsigned long long)w);
                        atomicAdd(&sh.h.cnt[d], 1u);
                    }
                });
                __syncthreads();
            }
            // thread t owns the bins BINS_PER_THREAD * t + j counted from the top
            uint64_t m[BINS_PER_THREAD], mine = 0;
            uint32_t c[BINS_PER_THREAD];
#pragma unroll
            for (int j = 0; j < BINS_PER_THREAD; ++j) {
                const int rb = BINS_PER_THREAD * tid + j;
                m[j] = rb < int(nb) ? sh.h.mass[nb - 1 - rb] : 0ull;
                c[j] = rb < int(nb) ? sh.h.cnt[nb - 1 - rb] : 0u;
                mine += m[j];
            }
            uint64_t total;
            const uint64_t excl = block_excl_scan<uint64_t>(mine, sh.wave_u64, &total);
            if (tid == 0) sh.best_rb = -1;
            __syncthreads();
            {   // the lowest of the thread's occupied bins whose first entry is still kept
                int mine_rb = -1;
                uint64_t run = excl;
#pragma unroll
                for (int j = 0; j < BINS_PER_THREAD; ++j) {
                    if (c[j] > 0 && before + run <= theta) mine_rb = BINS_PER_THREAD * tid + j;
                    run += m[j];
                }
                if (mine_rb >= 0) atomicMax(&sh.best_rb, mine_rb);
            }
            __syncthreads();
            const int best = sh.best_rb;
            {
                uint64_t run = excl;
#pragma unroll
                for (int j = 0; j < BINS_PER_THREAD; ++j) {
                    if (best == BINS_PER_THREAD * tid + j) { sh.sel_mass_above = run; sh.sel_mass = m[j]; sh.sel_count = c[j]; }
                    run += m[j];
                }
            }
            __syncthreads();
            prefix = (prefix << bits) | uint32_t(nb - 1 - best);
            before += sh.sel_mass_above;
            n_cut = sh.sel_count;
            m_cut = sh.sel_mass;
            __syncthreads();
        }
        kcut = prefix << level_shift<T>(LEVELS - 1);
        const uint64_t w_cut = n_cut ? m_cut / n_cut : 0;   // every entry of the tie group has this mass
        uint64_t r = n_cut;
        if (w_cut > 0) {
            const uint64_t fit = (theta - before) / w_cut + 1;  // entries t with before + t*w <= theta
            r = fit < r ? fit : r;
        }
        r_cut = uint32_t(r);
        z_kept = before + r * w_cut;
        if (r == n_cut) r_cut = 0xffffffffu;  // whole tie group survives: no rank bookkeeping needed
    }

    // ---- draw: first survivor, in index order, whose inclusive mass exceeds floor(u * Z) ----
    if constexpr (RADIX_ONLY) {
        if (vec) {
            draw_by_shares<T>(sh.ds, rp, vocab, temp, has_t, kmax, vmax, kcut, r_cut, u, out + row, lp_slot);
            return 1;
        }
    }
    const uint64_t tau = floor_scale(u, z_kept);
    const bool track_ties = r_cut != 0xffffffffu;
    if (tid == 0) sh.hit = -1;
    uint64_t carry_mass = 0;
    uint32_t carry_ties = 0;
    constexpr int TILE = S_THREADS * EPV;
    for (int tile = 0; tile < vocab; tile += TILE) {
        const int base = tile + tid * EPV;
        uint32_t keys[EPV];
        if (vec && base + EPV <= vocab) {
            const uint4 q = *reinterpret_cast<const uint4 *>(rp + base);
            const typename T::raw_t *e = reinterpret_cast<const typename T::raw_t *>(&q);
#pragma unroll
            for (int j = 0; j < EPV; ++j) keys[j] = elem_key<T>(e[j], temp, has_t);
        } else {
#pragma unroll
            for (int j = 0; j < EPV; ++j)
                keys[j] = (base + j < vocab) ? elem_key<T>(rp[base + j], temp, has_t) : 0u;
        }
        uint32_t tie_rank = 0;
        if (track_ties) {
            uint32_t c = 0;
#pragma unroll
            for (int j = 0; j < EPV; ++j) c += (base + j < vocab && keys[j] == kcut) ? 1u : 0u;
            uint32_t tot;
            tie_rank = carry_ties + block_excl_scan<uint32_t>(c, sh.wave_u32, &tot);
            carry_ties += tot;
        }
        uint64_t w[EPV];
        uint64_t msum = 0;
#pragma unroll
        for (int j = 0; j < EPV; ++j) {
            bool member = false;
            if (base + j < vocab) {
                if (keys[j] > kcut) member = true;
                else if (keys[j] == kcut && keys[j] >= kstar) member = !track_ties || (tie_rank++ < r_cut);
            }
            w[j] = member ? weight_fix(keys[j] == kmax ? 0.0f : value_of<T>(keys[j]) - vmax) : 0ull;
            msum += w[j];
        }
        uint64_t tot;
        const uint64_t excl = carry_mass + block_excl_scan<uint64_t>(msum, sh.wave_u64, &tot);
        if (excl <= tau && tau < excl + msum) {
            uint64_t cum = excl;
#pragma unroll
            for (int j = 0; j < EPV; ++j) {
                cum += w[j];
                if (cum > tau) { sh.hit = base + j; sh.pick_z = w[j]; break; }
            }
        }
        carry_mass += tot;
        if (carry_mass > tau) break;  // block-uniform: the hit lies in this tile
    }
    __syncthreads();
    if (tid == 0) {
        out[row] = sh.hit;
        if (lp_slot != nullptr) *lp_slot = sh.hit >= 0 ? log_ratio(sh.pick_z, z_kept) : __builtin_nanf("");
    }
    return 1;
}

// (512 threads: at most 128 registers, so that two workgroups fit a CU)
template <typename T, bool DENSE>
__global__ __launch_bounds__(S_THREADS) __attribute__((amdgpu_waves_per_eu(4, 4))) void sample_rows(const typename T::raw_t *__restrict__ logits,
                                                         int vocab, int64_t row_stride, SampleParams prm, int vec,
                                                         int no_fast) {
    // per-wavefront partial results of the row's log-sum-exp (its own few bytes of LDS: the routes' memory may still be
    // in use by a wavefront that finishes the row)
    __shared__ PolicyLse lse;
    const int done = sample_one_row<T, DENSE>(logits, vocab, row_stride, prm, vec, no_fast, lse);
    if (prm.out_policy != nullptr && done != 2) {
        // The route did not take the log-sum-exp along: one more pass over the row (from L2), by the whole block.
        const int64_t row = blockIdx.x;
        const typename T::raw_t *rp = logits + row * row_stride;
        row_lse_to_block<T>(rp, vocab, vec != 0, lse);
        __syncthreads();  // also: the id of the row is written (by thread 0, or by the wavefront that finished the row)
        if (threadIdx.x == 0) prm.out_policy[row] = lse.finish<T>(rp, prm.out_ids[row], vocab);
    }
}

}  // namespace
}  // namespace ka

#endif  // KA_SAMPLING_KERNEL_H

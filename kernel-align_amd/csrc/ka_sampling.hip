// Fused temperature -> top-k -> top-p -> draw, one workgroup per row.
//
// Every decision is taken on integers, so the sampled id does not depend on
// summation order, batch size or launch geometry:
//   * each scaled logit y maps to an order-preserving 32-bit key;
//   * the k-th largest key K* comes from an MSB-first radix descent over
//     2048-bin LDS count histograms (ties with K* survive, as in the reference);
//   * softmax masses are W(y - max) = trunc(2^40 * exp(y - max)), evaluated by a
//     fixed sequence of IEEE double operations, and summed as 64-bit integers;
//   * the top-p cut is a second radix descent over per-bin integer mass: it finds
//     the lowest key Kc whose first entry still has (mass before it) <= top_p * Z,
//     and how many entries r of the Kc tie group (ascending index) survive;
//   * the draw walks the row once more in index order with block-wide integer
//     prefix sums and stops at the first survivor whose inclusive mass exceeds
//     floor(u * Z_survivors).
// The row is re-read by every pass; after the first it comes from L2 / MALL.
// This radix path takes any row; shorter routes for common cases come first: the top-k candidate list
// (ka_sampling_topk.h: top_k <= 1024), and for 16-bit dtypes the no-filter and dense-histogram paths (ka_sampling_dense.h).
// For aligned fp32 rows outside the candidate list a variant of the kernel replaces the last pass by a draw
// over shares of the row (ka_sampling_draw.h).
#include <mutex>

#include "ka_sampling_common.h"
#include "ka_sampling_dense.h"
#include "ka_sampling_topk.h"
#include "ka_sampling_draw.h"

namespace ka {
namespace {

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
        if constexpr (!DENSE && T::kBytes == 2) {
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
            const int rb0 = 2 * tid, rb1 = 2 * tid + 1;
            const uint64_t m0 = rb0 < int(nb) ? sh.h.mass[nb - 1 - rb0] : 0ull;
            const uint64_t m1 = rb1 < int(nb) ? sh.h.mass[nb - 1 - rb1] : 0ull;
            const uint32_t c0 = rb0 < int(nb) ? sh.h.cnt[nb - 1 - rb0] : 0u;
            const uint32_t c1 = rb1 < int(nb) ? sh.h.cnt[nb - 1 - rb1] : 0u;
            uint64_t total;
            const uint64_t excl = block_excl_scan<uint64_t>(m0 + m1, sh.wave_u64, &total);
            if (tid == 0) sh.best_rb = -1;
            __syncthreads();
            const bool q0 = c0 > 0 && before + excl <= theta;
            const bool q1 = c1 > 0 && before + excl + m0 <= theta;
            if (q1) atomicMax(&sh.best_rb, rb1);
            else if (q0) atomicMax(&sh.best_rb, rb0);
            __syncthreads();
            const int best = sh.best_rb;
            if (best == rb0) { sh.sel_mass_above = excl; sh.sel_mass = m0; sh.sel_count = c0; }
            if (best == rb1) { sh.sel_mass_above = excl + m0; sh.sel_mass = m1; sh.sel_count = c1; }
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

template <typename T, bool DENSE>
__global__ __launch_bounds__(S_THREADS) void sample_rows(const typename T::raw_t *__restrict__ logits,
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
        LaneLse acc;
        for_each_raw<T>(rp, vocab, vec != 0, [&](int, typename T::raw_t raw) { acc.add(T::widen(raw)); });
        acc.to_block(lse);
        __syncthreads();  // also: the id of the row is written (by thread 0, or by the wavefront that finished the row)
        if (threadIdx.x == 0) prm.out_policy[row] = lse.finish<T>(rp, prm.out_ids[row], vocab);
    }
}

__global__ __launch_bounds__(256) void mass_fixed_kernel(const float *__restrict__ d, int64_t n, uint64_t *__restrict__ out) {
    const int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) out[i] = weight_fix(d[i]);
}

template <typename T>
int launch(const void *logits, int64_t batch, int64_t vocab, int64_t row_stride, const SampleParams &prm,
           void *workspace, size_t workspace_bytes, void *hip_stream, uint32_t flags = 0) {
    if (batch < 0) return fail(KA_ERR_BAD_ARG, "sample: batch %lld < 0", (long long)batch);
    if (batch == 0) return KA_OK;
    if (logits == nullptr || prm.uniforms == nullptr || prm.out_ids == nullptr)
        return fail(KA_ERR_BAD_ARG, "sample: null logits / uniforms / out_ids pointer");
    if (vocab < 1) return fail(KA_ERR_BAD_ARG, "sample: vocab %lld < 1", (long long)vocab);
    if (vocab >= (int64_t(1) << 22))
        return fail(KA_ERR_UNSUPPORTED, "sample: vocab %lld >= 2^22 (integer masses would overflow)",
                    (long long)vocab);
    if (row_stride < vocab) return fail(KA_ERR_BAD_ARG, "sample: row_stride < vocab");
    if (prm.temperature_rows == nullptr && !(prm.temperature > 0.0f))
        return fail(KA_ERR_BAD_ARG, "sample: temperature %g must be > 0", prm.temperature);
    if (prm.top_k_rows == nullptr && prm.top_k < 0) return fail(KA_ERR_BAD_ARG, "sample: top_k %d < 0", prm.top_k);
    if (prm.top_p_rows == nullptr && !(prm.top_p > 0.0f && prm.top_p <= 1.0f))
        return fail(KA_ERR_BAD_ARG, "sample: top_p %g outside (0, 1]", prm.top_p);
    if (batch >= (int64_t(1) << 31)) return fail(KA_ERR_UNSUPPORTED, "sample: batch too large");
    if (workspace_bytes < ka_sample_workspace_bytes(batch, vocab) || (workspace == nullptr && workspace_bytes > 0))
        return fail(KA_ERR_WORKSPACE, "sample: workspace of %zu B, need %zu B", workspace_bytes,
                    ka_sample_workspace_bytes(batch, vocab));
    const bool aligned = (reinterpret_cast<uintptr_t>(logits) % 16 == 0) && ((row_stride * T::kBytes) % 16 == 0);
    if (flags & ~uint32_t(KA_SAMPLE_FLAG_GENERAL_PATH | KA_SAMPLE_FLAG_BLOCK_WIDE_TOPK))
        return fail(KA_ERR_BAD_ARG, "sample: unknown flag bits 0x%x", flags);
    const bool no_fast = (flags & KA_SAMPLE_FLAG_GENERAL_PATH) != 0;
    const int path_bits = int(flags & 3u);
    // The dense-histogram path needs 157 KB of LDS (one workgroup per CU).  It serves top-p without top-k,
    // top_k > 1024 and no filter at all on aligned 16-bit rows; with per-row parameters any row may need it.
    bool dense = false;
    if (T::kBytes == 2 && aligned && !no_fast) {
        const bool per_row = prm.top_k_rows != nullptr || prm.top_p_rows != nullptr;
        const bool k_on = prm.top_k > 0 && prm.top_k < vocab;
        // (no filter at all: the histogram path for bf16; an fp16 row has too many distinct values for its list and
        //  takes the register-resident no-filter path of the small-LDS kernel)
        const bool no_filter = !k_on && !(prm.top_p < 1.0f);
        const bool fits_registers = vocab / 8 <= RES_VECS * S_THREADS;  // what the other kernel's no-filter path takes
        dense = per_row || (k_on && prm.top_k > S_THREADS) || (!k_on && !no_filter) ||
                (no_filter && (T::kDtype == KA_DTYPE_BF16 || !fits_registers));
    }
    hipStream_t stream = static_cast<hipStream_t>(hip_stream);
    const typename T::raw_t *lp = static_cast<const typename T::raw_t *>(logits);
    if constexpr (T::kBytes == 4) {
        // fp32 rows outside the top-k fast path (no filter, top-p alone, top_k > 1024): the radix path with the draw
        // done by shares of the row
        const bool per_row = prm.top_k_rows != nullptr || prm.top_p_rows != nullptr;
        const bool k_fast = prm.top_k > 0 && prm.top_k < vocab && prm.top_k <= S_THREADS;
        if (aligned && !per_row && !k_fast) {
            hipLaunchKernelGGL((sample_rows<T, true>), dim3(unsigned(batch)), dim3(S_THREADS), 0, stream, lp, int(vocab),
                               row_stride, prm, 1, path_bits);
            return check_hip(hipGetLastError(), "sample launch");
        }
    }
    if constexpr (T::kBytes == 2) {
      if (dense) {
        // the attribute belongs to the device: set once per device and dtype, not per call
        static std::mutex attr_mutex;
        static bool attr_set[64] = {};
        int device = 0;
        hipError_t rc = hipGetDevice(&device);
        if (rc != hipSuccess) return check_hip(rc, "sample: hipGetDevice");
        if (device < 0 || device >= 64) return fail(KA_ERR_UNSUPPORTED, "sample: device index %d", device);
        {
            std::lock_guard<std::mutex> lock(attr_mutex);
            if (!attr_set[device]) {
                rc = hipFuncSetAttribute(reinterpret_cast<const void *>(sample_rows<T, true>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, int(DENSE_LDS_BYTES));
                if (rc != hipSuccess) return check_hip(rc, "sample: reserving LDS for the dense-histogram path");
                attr_set[device] = true;
            }
        }
        hipLaunchKernelGGL((sample_rows<T, true>), dim3(unsigned(batch)), dim3(S_THREADS), DENSE_LDS_BYTES, stream, lp,
                           int(vocab), row_stride, prm, aligned ? 1 : 0, path_bits & 2);
        return check_hip(hipGetLastError(), "sample launch");
      }
    }
    hipLaunchKernelGGL((sample_rows<T, false>), dim3(unsigned(batch)), dim3(S_THREADS), 0, stream, lp, int(vocab),
                       row_stride, prm, aligned ? 1 : 0, path_bits);
    return check_hip(hipGetLastError(), "sample launch");
}

inline SampleParams scalar_params(float temperature, int32_t top_k, float top_p, const float *uniforms,
                                  int64_t *out_ids) {
    SampleParams p{};
    p.temperature = temperature;
    p.top_k = top_k;
    p.top_p = top_p;
    p.uniforms = uniforms;
    p.out_ids = out_ids;
    return p;
}

inline int launch_ex(int dtype, const void *logits, int64_t batch, int64_t vocab, int64_t row_stride,
                     const SampleParams &prm, void *workspace, size_t workspace_bytes, void *hip_stream, uint32_t flags) {
    switch (dtype) {
        case KA_DTYPE_BF16: return launch<Bf16>(logits, batch, vocab, row_stride, prm, workspace, workspace_bytes, hip_stream, flags);
        case KA_DTYPE_F16: return launch<F16>(logits, batch, vocab, row_stride, prm, workspace, workspace_bytes, hip_stream, flags);
        case KA_DTYPE_F32: return launch<F32>(logits, batch, vocab, row_stride, prm, workspace, workspace_bytes, hip_stream, flags);
        default: return fail(KA_ERR_BAD_ARG, "sample: unknown dtype code %d", dtype);
    }
}

}  // namespace
}  // namespace ka

// The kernels keep all their state in LDS and registers; the workspace argument is reserved.
KA_EXPORT size_t ka_sample_workspace_bytes(int64_t batch, int64_t vocab) {
    (void)batch;
    (void)vocab;
    return 0;
}

KA_EXPORT int ka_sample_topk_topp_bf16(const void *logits, int64_t batch, int64_t vocab, int64_t row_stride,
                                       float temperature, int32_t top_k, float top_p, const float *uniforms,
                                       int64_t *out_ids, void *workspace, size_t workspace_bytes,
                                       void *hip_stream) {
    return ka::launch<ka::Bf16>(logits, batch, vocab, row_stride,
                              ka::scalar_params(temperature, top_k, top_p, uniforms, out_ids), workspace,
                              workspace_bytes, hip_stream);
}
KA_EXPORT int ka_sample_topk_topp_f16(const void *logits, int64_t batch, int64_t vocab, int64_t row_stride,
                                      float temperature, int32_t top_k, float top_p, const float *uniforms,
                                      int64_t *out_ids, void *workspace, size_t workspace_bytes,
                                      void *hip_stream) {
    return ka::launch<ka::F16>(logits, batch, vocab, row_stride,
                              ka::scalar_params(temperature, top_k, top_p, uniforms, out_ids), workspace,
                              workspace_bytes, hip_stream);
}
KA_EXPORT int ka_sample_topk_topp_f32(const void *logits, int64_t batch, int64_t vocab, int64_t row_stride,
                                      float temperature, int32_t top_k, float top_p, const float *uniforms,
                                      int64_t *out_ids, void *workspace, size_t workspace_bytes,
                                      void *hip_stream) {
    return ka::launch<ka::F32>(logits, batch, vocab, row_stride,
                              ka::scalar_params(temperature, top_k, top_p, uniforms, out_ids), workspace,
                              workspace_bytes, hip_stream);
}

#ifdef KA_SAMPLE_STAMPS
KA_EXPORT int ka_debug_read_stamps(unsigned long long *host, int n) {
    return int(hipMemcpyFromSymbol(host, HIP_SYMBOL(ka::ka_dbg_stamps), size_t(n) * 8, 0, hipMemcpyDeviceToHost));
}
#endif

KA_EXPORT int ka_sample_mass_fixed(const float *d, int64_t n, uint64_t *out, void *hip_stream) {
    using namespace ka;
    if (n < 0) return fail(KA_ERR_BAD_ARG, "mass: n %lld < 0", (long long)n);
    if (n == 0) return KA_OK;
    if (d == nullptr || out == nullptr) return fail(KA_ERR_BAD_ARG, "mass: null pointer argument");
    if ((n + 255) / 256 >= (int64_t(1) << 31)) return fail(KA_ERR_UNSUPPORTED, "mass: n too large");
    hipLaunchKernelGGL(mass_fixed_kernel, dim3(unsigned((n + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(hip_stream), d, n, out);
    return check_hip(hipGetLastError(), "mass launch");
}

KA_EXPORT int ka_sample_ex(int dtype, const void *logits, int64_t batch, int64_t vocab, int64_t row_stride,
                           float temperature, const float *temperature_rows, int32_t top_k,
                           const int32_t *top_k_rows, float top_p, const float *top_p_rows, const float *uniforms,
                           int64_t *out_ids, float *out_logprob, float *out_policy_logprob, uint32_t flags,
                           void *workspace, size_t workspace_bytes, void *hip_stream) {
    ka::SampleParams p = ka::scalar_params(temperature, top_k, top_p, uniforms, out_ids);
    p.temperature_rows = temperature_rows;
    p.top_k_rows = top_k_rows;
    p.top_p_rows = top_p_rows;
    p.out_logprob = out_logprob;
    p.out_policy = out_policy_logprob;
    return ka::launch_ex(dtype, logits, batch, vocab, row_stride, p, workspace, workspace_bytes, hip_stream, flags);
}

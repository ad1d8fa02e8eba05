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
// (fast_topk), and for 16-bit dtypes the no-filter and dense-histogram paths further down.
#include <stdlib.h>

#include "ka_common.h"

namespace ka {
namespace {

constexpr int S_THREADS = 1024;
constexpr int S_WAVES = S_THREADS / kWave;
constexpr int BINS = 2048;
constexpr int FIX_BITS = 40;

// ---------------------------------------------------------------------------
// Scalar helpers (all exact)
// ---------------------------------------------------------------------------
__device__ __forceinline__ uint32_t key_of(float y) {
    const uint32_t b = __float_as_uint(y);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
// Keys of 16-bit dtypes keep only their significant top bits (a widened bf16 has 16, a widened fp16 19):
// negative values would otherwise carry ones in the unused low bits, and a key rebuilt from radix digits
// would not compare equal to the key of the element it came from.
template <typename T> __device__ __forceinline__ constexpr uint32_t key_mask() {
    return T::kDtype == KA_DTYPE_BF16 ? 0xffff0000u : (T::kDtype == KA_DTYPE_F16 ? 0xffffe000u : 0xffffffffu);
}
template <typename T> __device__ __forceinline__ uint32_t masked_key(float y) { return key_of(y) & key_mask<T>(); }
template <typename T> __device__ __forceinline__ float value_of(uint32_t key) {
    return __uint_as_float((key & 0x80000000u) ? (key & 0x7fffffffu) : (~key & key_mask<T>()));
}

// W(d) = trunc(2^40 * exp(d)), d <= 0, by a fixed sequence of IEEE double operations: one multiply for the
// range reduction, a degree-11 Horner evaluation with fused multiply-adds (Taylor coefficients 1/k!), one
// multiply by a power of two.  Contraction is off in this function, so exactly the operations written here
// are executed (the CPU statement of the operator performs the same ones, fma() included).  No branches: this
// runs for up to every entry of a row.
__device__ __forceinline__ uint64_t weight_fix(float d) {
#pragma clang fp contract(off)
    constexpr double C[12] = {0x1.0000000000000p+0,  0x1.0000000000000p+0,  0x1.0000000000000p-1,
                              0x1.5555555555555p-3,  0x1.5555555555555p-5,  0x1.1111111111111p-7,
                              0x1.6c16c16c16c17p-10, 0x1.a01a01a01a01ap-13, 0x1.a01a01a01a01ap-16,
                              0x1.71de3a556c734p-19, 0x1.27e4fb7789f5cp-22, 0x1.ae64567f544e4p-26};
    constexpr double LOG2E = 0x1.71547652b82fep+0, LN2 = 0x1.62e42fefa39efp-1;
    const double t = double(d) * LOG2E;
    const double tc = t < -64.0 ? -64.0 : t;  // keeps the conversion below in range; such t give 0 anyway
    const int n = int(tc - 0.5);
    const double f = tc - double(n);
    const double g = f * LN2;
    double p = C[11];
#pragma unroll
    for (int k = 10; k >= 0; --k) p = __builtin_fma(p, g, C[k]);
    const double scale = __longlong_as_double((long long)(uint64_t(1023 + FIX_BITS + n) << 52));
    // trunc(p * scale) < 2^42 as an integer: the low mantissa bits of trunc(.) + 2^52
    const uint64_t w = uint64_t(__double_as_longlong(__builtin_trunc(p * scale) + 0x1p52)) & 0x000fffffffffffffull;
    const uint64_t special = d > 0.0f ? (uint64_t(1) << FIX_BITS) : 0ull;  // d > 0 cannot occur; NaN -> 0
    return (d <= 0.0f && !(t < -41.0)) ? w : special;
}

// log(w / z) for integer masses, in fp64 (w >= 1: an entry of mass 0 is never drawn).
__device__ __forceinline__ float log_ratio(uint64_t w, uint64_t z) {
    return float(log(double(w)) - log(double(z)));
}

// floor(s * z) for an fp32 0 <= s < 1 and z < 2^62.
__device__ __forceinline__ uint64_t floor_scale(float s, uint64_t z) {
    const uint32_t b = __float_as_uint(s);
    const uint32_t e = (b >> 23) & 0xffu, m = b & 0x7fffffu;
    if (e == 0 && m == 0) return 0;
    uint64_t mant;
    int shift;
    if (e == 0) { mant = m; shift = 149; } else { mant = m | 0x800000u; shift = 150 - int(e); }
    const uint64_t lo = mant * z, hi = __umul64hi(mant, z);
    if (shift >= 128) return 0;
    if (shift >= 64) return hi >> (shift - 64);
    return (lo >> shift) | (hi << (64 - shift));  // 24 <= shift < 64
}

// y = x / T rounded to the logits dtype (torch's `logits / temperature`), -0 folded to +0.
template <typename T> struct Round;
template <> struct Round<Bf16> {
    static __device__ __forceinline__ float apply(float q) {
        uint32_t b = __float_as_uint(q);
        if ((b & 0x7fffffffu) > 0x7f800000u) return __uint_as_float(((b >> 16) | 0x40u) << 16);
        b += 0x7fffu + ((b >> 16) & 1u);
        return __uint_as_float(b & 0xffff0000u);
    }
    static constexpr int kLevels = 2;
};
template <> struct Round<F16> {
    static __device__ __forceinline__ float apply(float q) { return float(_Float16(q)); }
    static constexpr int kLevels = 2;
};
template <> struct Round<F32> {
    static __device__ __forceinline__ float apply(float q) { return q; }
    static constexpr int kLevels = 3;
};

// Radix levels, most significant first.  A widened bf16 occupies the top 16 key bits
// (1 + 8 + 7), a widened fp16 the top 19 (1 + 8 + 10), fp32 all 32.
template <typename T> __device__ __forceinline__ int level_shift(int level) {
    if (T::kDtype == KA_DTYPE_BF16) return level == 0 ? 21 : 16;
    if (T::kDtype == KA_DTYPE_F16) return level == 0 ? 21 : 13;
    return level == 0 ? 21 : (level == 1 ? 10 : 0);
}
template <typename T> __device__ __forceinline__ int level_bits(int level) {
    if (T::kDtype == KA_DTYPE_BF16) return level == 0 ? 11 : 5;
    if (T::kDtype == KA_DTYPE_F16) return level == 0 ? 11 : 8;
    return level == 2 ? 10 : 11;
}

template <typename T>
__device__ __forceinline__ uint32_t elem_key(typename T::raw_t raw, float temp, bool has_t) {
    float y = T::widen(raw);
    if (has_t) y = Round<T>::apply(y / temp);
    y = (y == 0.0f) ? 0.0f : y;
    y = (y != y) ? -__builtin_inff() : y;  // a NaN logit counts as -inf: it is never preferred to a number
    return masked_key<T>(y);
}

// ---------------------------------------------------------------------------
// Block-wide primitives (1024 threads, fixed exchange pattern)
// ---------------------------------------------------------------------------
constexpr int CAND_CAP = 1024;  // candidate slots of the top-k fast path (one per thread)

struct Histograms {
    uint32_t cnt[BINS];
    uint64_t mass[BINS];
};
struct Candidates {            // 24 KB, same footprint as the histograms
    uint32_t raw[CAND_CAP];    // element bits as loaded (widened to 32 bits)
    uint32_t idx[CAND_CAP];
    uint32_t skey[CAND_CAP];   // scaled keys in (key desc, index asc) order; first used for the thread maxima
    uint32_t sidx[CAND_CAP];
    uint64_t w[CAND_CAP];      // integer masses in that order
};

struct DenseScalars {
    uint64_t wave_u64[S_WAVES];
    uint32_t wave_u32[S_WAVES];
    uint64_t seg_mass[S_WAVES + 1];  // dense path: mass of each wavefront's share of the row, and of the ragged tail
    uint32_t seg_ties[S_WAVES + 1];  // ... and its number of tie-group entries
    uint64_t z_topk, before_cut, w_cut, pick_w;
    uint32_t i_topk, n_cut, kcut16, i_last, tie_hi, tie_lo, fail, n_inf;
    int best_i;
    int64_t hit;
};

struct alignas(16) Shared {
    union {
        Histograms h;
        Candidates c;
    };
    uint64_t wave_u64[S_WAVES];
    uint32_t wave_u32[S_WAVES];
    // broadcast slots
    uint32_t sel_digit, sel_above, sel_count;
    uint64_t sel_mass_above, sel_mass;
    int best_rb;
    uint32_t max_key;
    int64_t hit;
    uint32_t n_cand, pick_a, pick_b;
    uint64_t pick_z;
    DenseScalars ds;  // scalars of the resident no-filter path
};

template <typename V> __device__ __forceinline__ V shfl_up_v(V v, int off) { return __shfl_up(v, off, kWave); }

// Exclusive prefix sum over the block in thread order; *total = block sum.  Contains barriers.
template <typename V>
__device__ __forceinline__ V block_excl_scan(V v, V *wave_buf, V *total) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    V inc = v;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        const V t = shfl_up_v(inc, off);
        if (lane >= off) inc += t;
    }
    __syncthreads();  // wave_buf may still be read from a previous call
    if (lane == kWave - 1) wave_buf[wave] = inc;
    __syncthreads();
    V base = 0, sum = 0;
#pragma unroll
    for (int w = 0; w < S_WAVES; ++w) {
        const V x = wave_buf[w];
        if (w < wave) base += x;
        sum += x;
    }
    *total = sum;
    return base + inc - v;
}

__device__ __forceinline__ uint32_t block_max_u32(uint32_t v, Shared &sh) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const uint32_t t = __shfl_xor(v, off, kWave);
        v = t > v ? t : v;
    }
    __syncthreads();
    if ((threadIdx.x & (kWave - 1)) == 0) sh.wave_u32[threadIdx.x / kWave] = v;
    __syncthreads();
    uint32_t r = sh.wave_u32[0];
#pragma unroll
    for (int w = 1; w < S_WAVES; ++w) r = sh.wave_u32[w] > r ? sh.wave_u32[w] : r;
    return r;
}

// Finds the bin of sh.h.cnt[0 .. nb) that holds the rank-th largest entry (rank is 1-based, bins are ordered
// by digit, larger digit = larger keys).  Returns the digit; *above = entries in higher bins, *count =
// entries in the bin.  Every thread must call it; it contains barriers.
__device__ __forceinline__ uint32_t select_count_bin(Shared &sh, uint32_t nb, uint32_t rank, uint32_t *above,
                                                     uint32_t *count) {
    const int tid = threadIdx.x;
    // thread t owns the bins 2t and 2t+1 counted from the top
    const int rb0 = 2 * tid, rb1 = 2 * tid + 1;
    const uint32_t c0 = rb0 < int(nb) ? sh.h.cnt[nb - 1 - rb0] : 0u;
    const uint32_t c1 = rb1 < int(nb) ? sh.h.cnt[nb - 1 - rb1] : 0u;
    uint32_t total;
    const uint32_t excl = block_excl_scan<uint32_t>(c0 + c1, sh.wave_u32, &total);
    if (excl < rank && rank <= excl + c0) {
        sh.sel_digit = nb - 1 - rb0; sh.sel_above = excl; sh.sel_count = c0;
    } else if (excl + c0 < rank && rank <= excl + c0 + c1) {
        sh.sel_digit = nb - 1 - rb1; sh.sel_above = excl + c0; sh.sel_count = c1;
    }
    __syncthreads();
    const uint32_t digit = sh.sel_digit;
    *above = sh.sel_above;
    *count = sh.sel_count;
    __syncthreads();
    return digit;
}

__device__ __forceinline__ void clear_hist(Shared &sh) {
    for (int b = threadIdx.x; b < BINS; b += S_THREADS) {
        sh.h.cnt[b] = 0;
        sh.h.mass[b] = 0;
    }
}

// ---------------------------------------------------------------------------
// Row traversal: f(index, raw element) for every element, any order.
// ---------------------------------------------------------------------------
template <typename T, int U = 4, typename F>
__device__ __forceinline__ void for_each_raw(const typename T::raw_t *rp, int vocab, bool vec, F &&f) {
    constexpr int EPV = T::kPerVec;
    const int tid = threadIdx.x;
    if (vec) {
        const uint4 *vp = reinterpret_cast<const uint4 *>(rp);
        const int nvec = vocab / EPV;
        int v = tid;
        for (; v + (U - 1) * S_THREADS < nvec; v += U * S_THREADS) {
            uint4 q[U];
#pragma unroll
            for (int u = 0; u < U; ++u) q[u] = vp[v + u * S_THREADS];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const typename T::raw_t *e = reinterpret_cast<const typename T::raw_t *>(&q[u]);
#pragma unroll
                for (int j = 0; j < EPV; ++j) f((v + u * S_THREADS) * EPV + j, e[j]);
            }
        }
        for (; v < nvec; v += S_THREADS) {
            const uint4 q = vp[v];
            const typename T::raw_t *e = reinterpret_cast<const typename T::raw_t *>(&q);
#pragma unroll
            for (int j = 0; j < EPV; ++j) f(v * EPV + j, e[j]);
        }
        const int i = nvec * EPV + tid;
        if (i < vocab) f(i, rp[i]);
    } else {
        for (int i = tid; i < vocab; i += S_THREADS) f(i, rp[i]);
    }
}

// f(index, key of the scaled element).
template <typename T, typename F>
__device__ __forceinline__ void for_each_key(const typename T::raw_t *rp, int vocab, bool vec, float temp,
                                             bool has_t, F &&f) {
    for_each_raw<T>(rp, vocab, vec, [&](int i, typename T::raw_t raw) { f(i, elem_key<T>(raw, temp, has_t)); });
}

// Key of the raw (unscaled) element; the scaling x -> round(x / T) is monotone, so order statistics can be
// located on these keys and only the few candidates need the division.
template <typename T> __device__ __forceinline__ uint32_t raw_key(typename T::raw_t raw) {
    return masked_key<T>(T::widen(raw));
}
template <typename T> __device__ __forceinline__ typename T::raw_t raw_of_key(uint32_t key) {
    const uint32_t bits = __float_as_uint(value_of<T>(key));
    if (T::kDtype == KA_DTYPE_BF16) return typename T::raw_t(bits >> 16);
    if (T::kDtype == KA_DTYPE_F16) {
        union { _Float16 h; uint16_t u; } c;
        c.h = _Float16(value_of<T>(key));  // exact: the key came from a widened fp16
        return typename T::raw_t(c.u);
    }
    return typename T::raw_t(bits);
}
// Distance between neighbouring representable values in key space.
template <typename T> __device__ __forceinline__ uint32_t key_step() {
    return T::kDtype == KA_DTYPE_BF16 ? 0x10000u : (T::kDtype == KA_DTYPE_F16 ? 0x2000u : 1u);
}

// ---------------------------------------------------------------------------
// Top-k fast path: everything after the first read of the row happens on a short candidate list in LDS.
//
//   1. every lane takes the maximum raw key of its strided share of the row; the top_k-th largest of
//      those 1024 maxima, t, is a lower bound of the top_k-th largest element;
//   2. the bound is lowered to the smallest raw key that still scales to the same value as t (ties made
//      by the rounding of x / T must not be lost), and one more pass collects every element at or above
//      it: a superset of the top-k survivors, ~top_k + a few entries on ordinary rows;
//   3. the candidates are scaled, ranked by (key desc, index asc), cut by top-k (ties kept) and top-p on
//      integer masses, and the draw is taken over the survivors in index order.
// Returns false (having written nothing) when the candidates do not fit: the radix path then runs.
// All integer decisions are the same function of the row as in the radix path.
// ---------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ bool fast_topk(Shared &sh, const typename T::raw_t *rp, int vocab, bool vec, float temp,
                                          bool has_t, int top_k, bool use_p, float top_p, float u,
                                          int64_t *out_slot, float *lp_slot) {
    const int tid = threadIdx.x;
    // 1. lane maxima of the raw values (float max: one convert and half a v_max3 per element; which of
    //    -0 / +0 it returns does not matter, any lower bound of the top_k-th element will do)
    //    When the row fits (16-byte aligned, at most 16 vectors per lane: 131,072 bf16 entries) it is kept in
    //    registers, so that the collection pass below reads nothing from memory.
    constexpr int EPV = T::kPerVec;
    constexpr int RES_VECS = 16;
    const int nvec = vocab / EPV;
    const bool resident = vec && T::kDtype == KA_DTYPE_BF16 && nvec <= RES_VECS * S_THREADS;
    // A longer or wider row (fp32: up to 131,072 entries) does not fit in registers, but the maximum of each of
    // the lane's vectors does: the collection pass then re-reads only the few vectors that hold a candidate.
    constexpr int TRK_VECS = 32;
    const bool tracked = vec && !resident && nvec <= TRK_VECS * S_THREADS;
    uint4 held[RES_VECS];
    float vmaxs[TRK_VECS];
    float lmaxf = -__builtin_inff();
    if (tracked) {
        const uint4 *vp = reinterpret_cast<const uint4 *>(rp);
#pragma unroll
        for (int g = 0; g < TRK_VECS / 8; ++g) {
            uint4 q[8];
#pragma unroll
            for (int s = 0; s < 8; ++s) {
                const int v = tid + (g * 8 + s) * S_THREADS;
                q[s] = v < nvec ? vp[v] : make_uint4(0, 0, 0, 0);
            }
#pragma unroll
            for (int s = 0; s < 8; ++s) {
                float vm = -__builtin_inff();
                if (tid + (g * 8 + s) * S_THREADS < nvec) {
                    const typename T::raw_t *e = reinterpret_cast<const typename T::raw_t *>(&q[s]);
#pragma unroll
                    for (int j = 0; j < EPV; ++j) vm = fmaxf(vm, T::widen(e[j]));
                }
                vmaxs[g * 8 + s] = vm;
                lmaxf = fmaxf(lmaxf, vm);
            }
        }
        const int i = nvec * EPV + tid;  // ragged tail of the row
        if (i < vocab) lmaxf = fmaxf(lmaxf, T::widen(rp[i]));
    } else if (resident) {
        const uint4 *vp = reinterpret_cast<const uint4 *>(rp);
#pragma unroll
        for (int r = 0; r < RES_VECS; ++r) {
            const int v = tid + r * S_THREADS;
            held[r] = v < nvec ? vp[v] : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int r = 0; r < RES_VECS; ++r) {
            if (tid + r * S_THREADS < nvec) {
                const typename T::raw_t *e = reinterpret_cast<const typename T::raw_t *>(&held[r]);
#pragma unroll
                for (int j = 0; j < EPV; ++j) lmaxf = fmaxf(lmaxf, T::widen(e[j]));
            }
        }
        const int i = nvec * EPV + tid;  // ragged tail of the row
        if (i < vocab) lmaxf = fmaxf(lmaxf, T::widen(rp[i]));
    } else {
        for_each_raw<T, 8>(rp, vocab, vec, [&](int, typename T::raw_t raw) { lmaxf = fmaxf(lmaxf, T::widen(raw)); });
    }
    const uint32_t lmax = masked_key<T>(lmaxf);
    // the top_k-th largest of the 1024 lane maxima, by the same MSB-first descent over count histograms
    uint32_t bound = 0;
    {
        uint32_t rank = uint32_t(top_k), prefix = 0;
        for (int level = 0; level < Round<T>::kLevels; ++level) {
            const int shift = level_shift<T>(level), bits = level_bits<T>(level);
            const uint32_t nb = 1u << bits;
            __syncthreads();
            for (int b = tid; b < int(nb); b += S_THREADS) sh.h.cnt[b] = 0;
            __syncthreads();
            if (level == 0 || (lmax >> level_shift<T>(level - 1)) == prefix)
                atomicAdd(&sh.h.cnt[(lmax >> shift) & (nb - 1)], 1u);
            __syncthreads();
            uint32_t above, count;
            const uint32_t digit = select_count_bin(sh, nb, rank, &above, &count);
            prefix = (prefix << bits) | digit;
            rank -= above;
        }
        bound = prefix << level_shift<T>(Round<T>::kLevels - 1);
    }
    if (tid == 0) { sh.n_cand = 0; sh.hit = -1; }
    __syncthreads();
    // 2. widen the bound over the raw values that scale to the same value
    if (has_t) {
        const uint32_t ty = elem_key<T>(raw_of_key<T>(bound), temp, true);
        int guard = 0;
        while (bound >= key_step<T>() && guard < 64) {
            const uint32_t prev = bound - key_step<T>();
            if (elem_key<T>(raw_of_key<T>(prev), temp, true) < ty) break;
            bound = prev;
            ++guard;
        }
        if (guard == 64) return false;  // a huge temperature folds many values together: radix path
    }
    const float boundf = value_of<T>(bound);  // a float compare admits -0 next to +0: still a superset
    // Fewer than top_k lanes hold a number above -inf: the survivors then include -inf entries (and NaNs,
    // which count as -inf but fail every float compare).  Leave such rows to the radix path.
    if (boundf == -__builtin_inff()) return false;
    auto collect = [&](int i, typename T::raw_t raw) {
        if (T::widen(raw) >= boundf) {
            const uint32_t slot = atomicAdd(&sh.n_cand, 1u);
            if (slot < CAND_CAP) {
                sh.c.raw[slot] = uint32_t(raw);
                sh.c.idx[slot] = uint32_t(i);
            }
        }
    };
    if (resident) {
#pragma unroll
        for (int r = 0; r < RES_VECS; ++r) {
            const int v = tid + r * S_THREADS;
            if (v < nvec) {
                const typename T::raw_t *e = reinterpret_cast<const typename T::raw_t *>(&held[r]);
                float vm = T::widen(e[0]);
#pragma unroll
                for (int j = 1; j < EPV; ++j) vm = fmaxf(vm, T::widen(e[j]));
                if (vm >= boundf) {  // rare: about top_k vectors of the whole row hold a candidate
#pragma unroll
                    for (int j = 0; j < EPV; ++j) collect(v * EPV + j, e[j]);
                }
            }
        }
        const int i = nvec * EPV + tid;
        if (i < vocab) collect(i, rp[i]);
    } else if (tracked) {
        const uint4 *vp = reinterpret_cast<const uint4 *>(rp);
#pragma unroll
        for (int r = 0; r < TRK_VECS; ++r) {
            if (vmaxs[r] >= boundf) {  // rare: about top_k vectors of the whole row hold a candidate
                const int v = tid + r * S_THREADS;
                const uint4 q = vp[v];
                const typename T::raw_t *e = reinterpret_cast<const typename T::raw_t *>(&q);
#pragma unroll
                for (int j = 0; j < EPV; ++j) collect(v * EPV + j, e[j]);
            }
        }
        const int i = nvec * EPV + tid;
        if (i < vocab) collect(i, rp[i]);
    } else {
        for_each_raw<T, 8>(rp, vocab, vec, collect);
    }
    __syncthreads();
    const uint32_t nc = sh.n_cand;
    if (nc > CAND_CAP) return false;
    // 3a. scale the candidates and rank them by (key desc, index asc)
    uint32_t my_key = 0, my_idx = 0;
    if (tid < int(nc)) {
        my_key = elem_key<T>(typename T::raw_t(sh.c.raw[tid]), temp, has_t);
        my_idx = sh.c.idx[tid];
    }
    __syncthreads();
    if (tid < int(nc)) sh.c.raw[tid] = my_key;  // raw[] now holds the scaled keys, unsorted
    uint32_t *const rank_of = reinterpret_cast<uint32_t *>(sh.c.w);  // scratch until the masses are written
    if (tid < kWave) rank_of[tid] = 0;
    __syncthreads();
    if (nc <= kWave) {
        // short list (the ordinary case): candidate i = lane, wavefront w counts against entries 4w .. 4w+3
        const int i = tid & (kWave - 1), j0 = (tid / kWave) * 4;
        if (i < int(nc) && j0 < int(nc)) {
            const uint32_t ki = sh.c.raw[i], ii = sh.c.idx[i];
            uint32_t part = 0;
#pragma unroll
            for (int j = j0; j < j0 + 4; ++j)
                if (j < int(nc)) {
                    const uint32_t kj = sh.c.raw[j], ij = sh.c.idx[j];
                    part += (kj > ki || (kj == ki && ij < ii)) ? 1u : 0u;
                }
            if (part) atomicAdd(&rank_of[i], part);
        }
        __syncthreads();
        if (tid < int(nc)) {
            const uint32_t rank = rank_of[tid];
            sh.c.skey[rank] = my_key;
            sh.c.sidx[rank] = my_idx;
        }
    } else if (tid < int(nc)) {
        uint32_t rank = 0;
        for (uint32_t j = 0; j < nc; ++j) {
            const uint32_t kj = sh.c.raw[j], ij = sh.c.idx[j];
            rank += (kj > my_key || (kj == my_key && ij < my_idx)) ? 1u : 0u;
        }
        sh.c.skey[rank] = my_key;
        sh.c.sidx[rank] = my_idx;
    }
    __syncthreads();
    // 3b. top-k with ties: survivors are the sorted prefix with key >= key of position top_k - 1
    const uint32_t kmax = sh.c.skey[0];
    const float vmax = value_of<T>(kmax);
    const uint32_t kstar = sh.c.skey[top_k - 1];
    if (tid < int(nc) && sh.c.skey[tid] >= kstar && (tid + 1 == int(nc) || sh.c.skey[tid + 1] < kstar))
        sh.pick_b = uint32_t(tid) + 1;
    __syncthreads();
    const uint32_t na = sh.pick_b;
    // 3c. integer masses, exclusive prefix in sorted order, top-p cut
    uint64_t w = 0;
    if (tid < int(na)) {
        const uint32_t k = sh.c.skey[tid];
        w = weight_fix(k == kmax ? 0.0f : value_of<T>(k) - vmax);
        sh.c.w[tid] = w;
    }
    uint64_t z_topk;
    const uint64_t before = block_excl_scan<uint64_t>(w, sh.wave_u64, &z_topk);
    uint32_t nb = na;
    uint64_t z_kept = z_topk;
    if (use_p) {
        const uint64_t theta = floor_scale(top_p, z_topk);
        const bool kept = tid < int(na) && before <= theta;
        // `before` is non-decreasing along the sorted order, so the survivors are a prefix; its last lane
        // publishes the count and the surviving mass
        const uint64_t next_before = before + w;
        if (kept && (tid + 1 == int(na) || next_before > theta)) {
            sh.pick_a = uint32_t(tid) + 1;
            sh.pick_z = next_before;
        }
        __syncthreads();
        nb = sh.pick_a;
        z_kept = sh.pick_z;
    }
    // 3d. draw: inclusive mass over the survivors in index order; the first index above floor(u * Z) wins
    const uint64_t tau = floor_scale(u, z_kept);
    if (tid < int(nb)) {
        const uint32_t mine = sh.c.sidx[tid];
        uint64_t cum = 0;
        for (uint32_t j = 0; j < nb; ++j) cum += sh.c.sidx[j] <= mine ? sh.c.w[j] : 0ull;
        if (cum > tau) atomicMin(reinterpret_cast<unsigned long long *>(&sh.hit), (unsigned long long)mine);
    }
    __syncthreads();
    if (tid == 0) *out_slot = sh.hit;
    if (lp_slot != nullptr && tid < int(nb) && int64_t(sh.c.sidx[tid]) == sh.hit) *lp_slot = log_ratio(sh.c.w[tid], z_kept);
    return true;
}


// ---------------------------------------------------------------------------
// Paths for 16-bit dtypes (bf16, fp16), rows of at most 131,072 entries, 16-byte aligned.
// Since a 16-bit dtype has only 65,536 values, an entry's integer mass is a function of its 16-bit key.
//
//   no filter   : the row is read once into registers (16 x uint4 per lane, a contiguous run of entries per
//                 lane) and every entry is replaced by the key of its scaled value; one pass evaluates every
//                 entry's mass, one block-wide prefix sum of the lane totals finds the lane that holds the
//                 draw, which then finds the vector and the entry.
//   dense path  : (top-p without top-k, or top_k > 1024) a count histogram over all 65,536 raw keys in LDS
//                 (16-bit counters, two per word) is filled by one streaming pass and compacted into a list
//                 of the occupied keys in descending order; temperature and masses are applied once per
//                 occupied key (a few thousand instead of 128 K; runs of keys that scale to one value form
//                 one tie group); prefix sums over the list give the top-k key, Z, the top-p cut and the
//                 surviving mass; the masses of the surviving keys go into a table indexed by
//                 key - lowest surviving key, and the draw streams the row twice more (from L2 / MALL):
//                 per-wavefront masses first, then the step, lane and entry inside one wavefront's share.
// Both return false (having written no output) when a row does not fit (a counter overflow, too many occupied
// keys, survivors spanning too many keys, a temperature that folds more than 64 values into one); the radix
// path then runs.  All integer decisions are the same function of the row as in the radix path.
// ---------------------------------------------------------------------------
constexpr int RES_VECS = 16;
constexpr int D_WORDS = 32768;              // 65,536 16-bit counters
constexpr int D_LIST_CAP = 7168;            // occupied keys the list can hold (4 B each)
constexpr int D_TABLE_CAP = D_LIST_CAP / 2; // keys spanned by the survivors (8 B each, same LDS region)
constexpr int D_PER_THREAD = D_LIST_CAP / S_THREADS;  // list entries per thread

constexpr size_t DENSE_LDS_BYTES = size_t(D_WORDS) * 4 + size_t(D_LIST_CAP) * 4 + sizeof(DenseScalars);

template <typename T> __device__ __forceinline__ uint32_t key16_of(float y) {  // y is a value of the dtype
    if (T::kDtype == KA_DTYPE_BF16) return masked_key<T>(y) >> 16;
    union { _Float16 h; uint16_t u; } c;
    c.h = _Float16(y);
    return (c.u & 0x8000u) ? (~uint32_t(c.u) & 0xffffu) : (uint32_t(c.u) | 0x8000u);
}
template <typename T> __device__ __forceinline__ float value_of_key16(uint32_t k) {
    if (T::kDtype == KA_DTYPE_BF16) return value_of<T>(k << 16);
    union { _Float16 h; uint16_t u; } c;
    c.u = uint16_t((k & 0x8000u) ? (k & 0x7fffu) : (~k & 0xffffu));
    return float(c.h);
}
// 16-bit key of the scaled entry (temperature, -0 -> +0, NaN -> -inf), computed on the 16-bit patterns with
// selects only: this runs once per entry of the row.
template <typename T, bool HAS_T>
__device__ __forceinline__ uint32_t elem_key16(uint32_t raw, float temp) {
    uint32_t h = raw;  // 16-bit pattern of the scaled value
    if (HAS_T) {
        const float q = T::widen(typename T::raw_t(raw)) / temp;
        if (T::kDtype == KA_DTYPE_BF16) {
            const uint32_t b = __float_as_uint(q);
            // round to nearest even on the upper 16 bits; +-inf stays, a NaN is replaced below
            h = ((b + 0x7fffu + ((b >> 16) & 1u)) >> 16) | (((b & 0x7fffffffu) > 0x7f800000u) ? 0x7fc0u : 0u);
        } else {
            union { _Float16 f; uint16_t u; } c;
            c.f = _Float16(q);
            h = c.u;
        }
    }
    constexpr uint32_t kInf = T::kDtype == KA_DTYPE_BF16 ? 0x7f80u : 0x7c00u;
    const uint32_t mag = h & 0x7fffu;
    h = mag == 0 ? 0u : h;                        // -0 -> +0
    h = mag > kInf ? (0x8000u | kInf) : h;        // NaN -> -inf
    return (h & 0x8000u) ? (~h & 0xffffu) : (h | 0x8000u);
}

__device__ __forceinline__ uint64_t wave_sum_u64(uint64_t v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}
__device__ __forceinline__ uint32_t block_max_u32_buf(uint32_t v, uint32_t *wave_buf) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const uint32_t t = __shfl_xor(v, off, kWave);
        v = t > v ? t : v;
    }
    __syncthreads();
    if ((threadIdx.x & (kWave - 1)) == 0) wave_buf[threadIdx.x / kWave] = v;
    __syncthreads();
    uint32_t r = wave_buf[0];
#pragma unroll
    for (int w = 1; w < S_WAVES; ++w) r = wave_buf[w] > r ? wave_buf[w] : r;
    return r;
}

// Layout of a resident row: lane t owns the vectors [t * vpl, (t + 1) * vpl) (vpl = ceil(nvec / 1024) <= 16),
// a contiguous run of entries, so index order is (lane, vector, entry) and one block-wide prefix sum over
// per-lane totals finds the lane that holds the draw.  (The loads are 16 bytes per lane at a stride of
// 16 * vpl bytes; the lines are shared by the lane's consecutive loads and come from L1 / L2.)
__device__ __forceinline__ bool lane_has_vec(int r, int vpl, int nvec) {
    return r < vpl && int(threadIdx.x) * vpl + r < nvec;
}

// The draw over a resident row of 16-bit keys: mass(key) gives an entry's integer mass (0 for an entry that
// did not survive the filters); every sum is an integer sum.
// With `ties` set, only the first r_cut entries (in index order) equal to tie_key survive, each with mass
// w_tie; mass() must then return 0 for tie_key.
// HEAVY = mass() is a long instruction sequence (a polynomial in fp64): the per-entry loops then stay rolled,
// four entries per iteration for instruction-level parallelism, because 128 inlined copies would not fit the
// instruction cache.  A cheap mass() (an LDS lookup) is fully unrolled.
template <bool HEAVY, typename F>
__device__ __forceinline__ void resident_draw(DenseScalars &ds, const uint4 (&held)[RES_VECS], int vpl, int nvec,
                                              uint32_t tail_key, bool has_tail, int tail_index, bool any_tail,
                                              float u, bool ties, uint32_t tie_key, uint32_t r_cut, uint64_t w_tie,
                                              F &&mass, int64_t *out_slot, float *lp_slot) {
    const int tid = threadIdx.x;
    if (tid == 0) ds.hit = -1;
    // mass of one vector without its tie-group entries, and the number of those
    auto vec_mass = [&](const uint4 &v) -> uint64_t {
        uint64_t w8 = 0;
        if constexpr (HEAVY) {
#pragma unroll 1
            for (int half = 0; half < 2; ++half) {
                const uint32_t lo = half ? v.z : v.x, hi = half ? v.w : v.y;
                w8 += (mass(lo & 0xffffu) + mass(lo >> 16)) + (mass(hi & 0xffffu) + mass(hi >> 16));
            }
        } else {
            const uint32_t in[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int q = 0; q < 4; ++q) w8 += mass(in[q] & 0xffffu) + mass(in[q] >> 16);
        }
        return w8;
    };
    auto vec_ties = [&](const uint4 &v) -> uint32_t {
        const uint32_t in[4] = {v.x, v.y, v.z, v.w};
        uint32_t t = 0;
#pragma unroll
        for (int q = 0; q < 4; ++q) t += (((in[q] & 0xffffu) == tie_key) ? 1u : 0u) + (((in[q] >> 16) == tie_key) ? 1u : 0u);
        return ties ? t : 0u;
    };
    // ---- masses of this lane in four groups of four vectors, tie-group entries of the lane ---------------------
    uint64_t gsum[4] = {0, 0, 0, 0};
    uint32_t lane_ties = 0;
#pragma unroll
    for (int r = 0; r < RES_VECS; ++r) {
        if (lane_has_vec(r, vpl, nvec)) {
            gsum[r >> 2] += vec_mass(held[r]);
            lane_ties += vec_ties(held[r]);
        }
    }
    // ---- lane totals in index order ----------------------------------------------------------------------------
    uint32_t first_rank = 0, all_vec_ties = 0;  // rank of the lane's first tie-group entry; such entries in all vectors
    if (ties) first_rank = block_excl_scan<uint32_t>(lane_ties, ds.wave_u32, &all_vec_ties);
    const uint32_t lane_room = first_rank < r_cut ? r_cut - first_rank : 0u;
    const uint64_t lane_total = (gsum[0] + gsum[1]) + (gsum[2] + gsum[3]) +
                                uint64_t(lane_ties < lane_room ? lane_ties : lane_room) * w_tie;
    uint64_t z_vec;
    const uint64_t lane_before = block_excl_scan<uint64_t>(lane_total, ds.wave_u64, &z_vec);
    // the ragged tail of the row (fewer than 8 entries after the last vector, one per lane of wavefront 0)
    uint64_t tail_mass = 0, tail_before = 0, z_tail = 0;
    if (any_tail) {
        uint32_t tail_rank = 0, tot_t;
        const bool tail_tie = ties && has_tail && tail_key == tie_key;
        if (ties) tail_rank = all_vec_ties + block_excl_scan<uint32_t>(tail_tie ? 1u : 0u, ds.wave_u32, &tot_t);
        if (has_tail) tail_mass = tail_tie ? (tail_rank < r_cut ? w_tie : 0ull) : mass(tail_key);
        tail_before = z_vec + block_excl_scan<uint64_t>(tail_mass, ds.wave_u64, &z_tail);
    }
    const uint64_t z = z_vec + z_tail;
    const uint64_t tau = floor_scale(u, z);
    // ---- the lane that holds tau finds the group, the vector, the entry ------------------------------------------
    // (vectors are picked with masks: a chain of selects on a run-time index would be turned into a dynamically
    // indexed load and move the sixteen vectors to scratch memory)
    if (lane_before <= tau && tau < lane_before + lane_total) {
        uint64_t cum = lane_before;
        uint32_t rank = first_rank;
        uint4 c4[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) c4[i] = make_uint4(0, 0, 0, 0);
        int g_hit = -1;
        uint64_t cum_g = 0;
        uint32_t rank_g = 0;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            uint32_t tg = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (lane_has_vec(g * 4 + i, vpl, nvec)) tg += vec_ties(held[g * 4 + i]);
            const uint32_t room = rank < r_cut ? r_cut - rank : 0u;
            const uint64_t gt = gsum[g] + uint64_t(tg < room ? tg : room) * w_tie;
            const bool here = g_hit < 0 && tau < cum + gt;
            const uint32_t m = here ? 0xffffffffu : 0u;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                c4[i].x |= held[g * 4 + i].x & m;
                c4[i].y |= held[g * 4 + i].y & m;
                c4[i].z |= held[g * 4 + i].z & m;
                c4[i].w |= held[g * 4 + i].w & m;
            }
            if (here) { g_hit = g; cum_g = cum; rank_g = rank; }
            cum += gt;
            rank += tg;
        }
        uint4 cur = make_uint4(0, 0, 0, 0);
        int r_hit = -1;
        uint64_t cum_v = 0;
        uint32_t rank_v = 0;
        cum = cum_g;
        rank = rank_g;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const bool present = lane_has_vec(g_hit * 4 + i, vpl, nvec);
            const uint32_t tv = present ? vec_ties(c4[i]) : 0u;
            const uint32_t room = rank < r_cut ? r_cut - rank : 0u;
            const uint64_t vt = (present ? vec_mass(c4[i]) : 0ull) + uint64_t(tv < room ? tv : room) * w_tie;
            const bool here = r_hit < 0 && tau < cum + vt;
            const uint32_t m = here ? 0xffffffffu : 0u;
            cur.x |= c4[i].x & m;
            cur.y |= c4[i].y & m;
            cur.z |= c4[i].z & m;
            cur.w |= c4[i].w & m;
            if (here) { r_hit = g_hit * 4 + i; cum_v = cum; rank_v = rank; }
            cum += vt;
            rank += tv;
        }
        uint64_t c2 = cum_v;
        uint32_t rk = rank_v;
#pragma unroll 1
        for (int j = 0; j < 8; ++j) {
            const uint32_t word = j < 4 ? (j < 2 ? cur.x : cur.y) : (j < 6 ? cur.z : cur.w);
            const uint32_t k = (word >> ((j & 1) * 16)) & 0xffffu;
            const uint64_t wj = (ties && k == tie_key) ? ((rk++ < r_cut) ? w_tie : 0ull) : mass(k);
            c2 += wj;
            if (c2 > tau) { ds.hit = (tid * vpl + r_hit) * 8 + j; ds.pick_w = wj; break; }
        }
    }
    if (any_tail && has_tail && tail_before <= tau && tau < tail_before + tail_mass) {
        ds.hit = tail_index;
        ds.pick_w = tail_mass;
    }
    __syncthreads();
    if (tid == 0) {
        *out_slot = ds.hit;
        if (lp_slot != nullptr) *lp_slot = ds.hit >= 0 ? log_ratio(ds.pick_w, z) : __builtin_nanf("");
    }
}

// Reads the row into registers as 16-bit keys of the scaled entries; returns the lane's largest key.
template <typename T, bool HAS_T>
__device__ __forceinline__ uint32_t resident_load_keys_t(const typename T::raw_t *rp, int vocab, int vpl, int nvec,
                                                         float temp, uint4 (&held)[RES_VECS], uint32_t *tail_key,
                                                         bool *has_tail) {
    const int tid = threadIdx.x;
    const uint4 *vp = reinterpret_cast<const uint4 *>(rp) + tid * vpl;
#pragma unroll
    for (int r = 0; r < RES_VECS; ++r) held[r] = lane_has_vec(r, vpl, nvec) ? vp[r] : make_uint4(0, 0, 0, 0);
    uint32_t kmax = 0;
#pragma unroll
    for (int r = 0; r < RES_VECS; ++r) {
        if (lane_has_vec(r, vpl, nvec)) {
            // explicit shifts (no 16-bit pointer accesses): the vectors must stay in registers
            const uint32_t in[4] = {held[r].x, held[r].y, held[r].z, held[r].w};
            uint32_t o[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint32_t k0 = elem_key16<T, HAS_T>(in[q] & 0xffffu, temp);
                const uint32_t k1 = elem_key16<T, HAS_T>(in[q] >> 16, temp);
                o[q] = k0 | (k1 << 16);
                kmax = k0 > kmax ? k0 : kmax;
                kmax = k1 > kmax ? k1 : kmax;
            }
            held[r] = make_uint4(o[0], o[1], o[2], o[3]);
        }
    }
    const int i = nvec * 8 + tid;
    *has_tail = i < vocab;
    *tail_key = *has_tail ? elem_key16<T, HAS_T>(uint32_t(rp[i]), temp) : 0u;
    if (*has_tail) kmax = *tail_key > kmax ? *tail_key : kmax;
    return kmax;
}
template <typename T>
__device__ __forceinline__ uint32_t resident_load_keys(const typename T::raw_t *rp, int vocab, int vpl, int nvec,
                                                       float temp, bool has_t, uint4 (&held)[RES_VECS],
                                                       uint32_t *tail_key, bool *has_tail) {
    return has_t ? resident_load_keys_t<T, true>(rp, vocab, vpl, nvec, temp, held, tail_key, has_tail)
                 : resident_load_keys_t<T, false>(rp, vocab, vpl, nvec, temp, held, tail_key, has_tail);
}

template <typename T>
__device__ __forceinline__ bool resident_ok(int vocab, bool vec) {
    return vec && T::kBytes == 2 && vocab / 8 <= RES_VECS * S_THREADS;
}

// No filter at all: every entry survives.
template <typename T>
__device__ __forceinline__ bool nofilter_resident(DenseScalars &ds, const typename T::raw_t *rp, int vocab, bool vec,
                                                  float temp, bool has_t, float u, int64_t *out_slot, float *lp_slot) {
    if (!resident_ok<T>(vocab, vec)) return false;
    const int nvec = vocab / 8;
    uint4 held[RES_VECS];
    uint32_t tail_key;
    bool has_tail;
    const int vpl = (nvec + S_THREADS - 1) / S_THREADS;
    const uint32_t lmax = resident_load_keys<T>(rp, vocab, vpl, nvec, temp, has_t, held, &tail_key, &has_tail);
    const uint32_t kmax = block_max_u32_buf(lmax, ds.wave_u32);
    const float vmax = value_of_key16<T>(kmax);
    resident_draw<true>(ds, held, vpl, nvec, tail_key, has_tail, nvec * 8 + int(threadIdx.x), vocab != nvec * 8, u, false,
                        0u, 0xffffffffu, 0ull,
                  [&](uint32_t k) { return weight_fix(k == kmax ? 0.0f : value_of_key16<T>(k) - vmax); }, out_slot,
                  lp_slot);
    return true;
}

// Word w of the count histogram holds the keys 2w (low half) and 2w + 1 (high half).  A lane later reads
// 32 consecutive words (128 B) with ds_read_b128; the 16-byte chunk index inside each 128-byte block is
// XOR-swizzled with the block index so that those reads spread over the banks.
__device__ __forceinline__ int hist_slot(int word) {
    return word ^ ((word >> 4) & 0x1c);  // chunk index (bits 2..4) ^= bits 1..3 of the block index (bits 6..8)
}

// Walks the vectors of this wavefront's share of the row: wavefront w owns the vectors [w * vpw, (w + 1) * vpw)
// (a contiguous sixteenth of the row, so index order is (wavefront, step, lane, entry)), lane l takes the
// vectors l, l + 64, ... of that share: every load instruction covers 1 KB of consecutive memory.  Calls
// f(valid, plain, keys) once per step with the eight 16-bit keys of the lane's vector (plain: none of them is a
// zero, an infinity or a NaN); the trip count is the same for all lanes, so f may contain wavefront-wide
// exchanges.  Four loads are in flight per lane.
template <typename T, bool HAS_T, typename F>
__device__ __forceinline__ void for_wave_vectors(const uint4 *vp, int n_here, float temp, F &&f) {
    const int lane = threadIdx.x & (kWave - 1);
#pragma unroll 1
    for (int i0 = 0; i0 < n_here; i0 += 4 * kWave) {
        uint4 q[4];
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const int idx = i0 + s * kWave + lane;
            q[s] = idx < n_here ? vp[idx] : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            if (i0 + s * kWave < n_here) {  // wavefront-uniform
                const uint32_t in[4] = {q[s].x, q[s].y, q[s].z, q[s].w};
                uint32_t k[8];
                bool plain = false;  // no zero, infinity or NaN in the vector: two keys per instruction, no selects
                if constexpr (!HAS_T) {
                    constexpr uint32_t kAdd = T::kDtype == KA_DTYPE_BF16 ? 0x00800080u : 0x04000400u;
                    uint32_t special = 0;
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        const uint32_t mag = in[c] & 0x7fff7fffu;
                        // bit 15 of a half: set by (mag + kAdd) when its exponent field is all ones; cleared in
                        // ((mag | 0x8000) - 1) when the half is zero (bit 15 also stops the borrow)
                        special |= (mag + kAdd) | ~((mag | 0x80008000u) - 0x00010001u);
                    }
                    plain = (special & 0x80008000u) == 0;
                }
                if (plain) {
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        const uint32_t neg = ((in[c] >> 15) & 0x00010001u) * 0xffffu;  // 0xffff in each negative half
                        const uint32_t kk = in[c] ^ (neg | 0x80008000u);
                        k[2 * c] = kk & 0xffffu;
                        k[2 * c + 1] = kk >> 16;
                    }
                } else {
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        k[2 * c] = elem_key16<T, HAS_T>(in[c] & 0xffffu, temp);
                        k[2 * c + 1] = elem_key16<T, HAS_T>(in[c] >> 16, temp);
                    }
                }
                f(i0 + s * kWave + lane < n_here, plain, k);
            }
        }
    }
}

__device__ __forceinline__ uint32_t wave_sum_u32(uint32_t v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}
// Exclusive prefix sums over the 64 lanes of a wavefront.
template <typename V> __device__ __forceinline__ V wave_excl_scan(V v) {
    const int lane = threadIdx.x & (kWave - 1);
    V inc = v;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        const V t = __shfl_up(inc, off, kWave);
        if (lane >= off) inc += t;
    }
    return inc - v;
}

template <typename T, bool HAS_T, bool ALL_SURVIVE>
__device__ __forceinline__ bool dense_stream(unsigned char *lds, const typename T::raw_t *rp, int vocab, bool vec,
                                             float temp, bool use_k, int top_k, bool use_p, float top_p, float u,
                                             int64_t *out_slot, float *lp_slot) {
    if (!resident_ok<T>(vocab, vec)) return false;
    uint32_t *hist = reinterpret_cast<uint32_t *>(lds);
    uint32_t *list = hist + D_WORDS;                                   // (key << 16) | count, descending keys
    uint64_t *table = reinterpret_cast<uint64_t *>(list);              // later: mass of key kcut16 + i
    DenseScalars &ds = *reinterpret_cast<DenseScalars *>(list + D_LIST_CAP);
    const int tid = threadIdx.x;
    const int wave = tid / kWave;
    constexpr bool all_survive = ALL_SURVIVE;  // no filter at all (the caller passes use_k = use_p = false)
    const int nvec = vocab / 8;
    const int vpw = (nvec + S_WAVES - 1) / S_WAVES;                    // vectors per wavefront
    const int v0 = wave * vpw;
    const int n_here = nvec - v0 < vpw ? (nvec - v0 > 0 ? nvec - v0 : 0) : vpw;
    const uint4 *vp = reinterpret_cast<const uint4 *>(rp) + v0;
    // the ragged tail of the row: fewer than 8 entries after the last vector, one per lane of wavefront 0
    const int tail_index = nvec * 8 + tid;
    const bool has_tail = tail_index < vocab;
    const uint32_t tail_key = has_tail ? elem_key16<T, false>(uint32_t(rp[tail_index]), 1.0f) : 0u;

    // ---- 1. counts of the raw keys (no temperature yet: the scaling x -> round(x / T) is monotone, so it can be
    //         applied to the few thousand occupied keys instead of to every entry) into the histogram ----------
    {
        uint4 *h4 = reinterpret_cast<uint4 *>(hist);
        for (int i = tid; i < D_WORDS / 4; i += S_THREADS) h4[i] = make_uint4(0, 0, 0, 0);
    }
    __syncthreads();
    // Entries at -inf (a masked vocabulary; NaNs count as -inf) have mass 0 unless the whole row is -inf: they are
    // counted apart in 32 bits and take no further part, so that a row with more than 65,535 masked entries does
    // not overflow a 16-bit counter.
    constexpr uint32_t kNegInfKey = ~(0x8000u | (T::kDtype == KA_DTYPE_BF16 ? 0x7f80u : 0x7c00u)) & 0xffffu;
    if (tid == 0) ds.n_inf = 0;
    uint32_t lmax = tail_key;
    uint32_t my_inf = (has_tail && tail_key == kNegInfKey) ? 1u : 0u;
    for_wave_vectors<T, false>(vp, n_here, 1.0f, [&](bool valid, bool plain, const uint32_t (&k)[8]) {
        if (valid && plain) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                atomicAdd(&hist[hist_slot(k[j] >> 1)], (k[j] & 1) ? 0x10000u : 1u);
                lmax = k[j] > lmax ? k[j] : lmax;
            }
        } else if (valid) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                if (k[j] == kNegInfKey) ++my_inf;
                else atomicAdd(&hist[hist_slot(k[j] >> 1)], (k[j] & 1) ? 0x10000u : 1u);
                lmax = k[j] > lmax ? k[j] : lmax;
            }
        }
    });
    if (has_tail && tail_key != kNegInfKey) atomicAdd(&hist[hist_slot(tail_key >> 1)], (tail_key & 1) ? 0x10000u : 1u);
    my_inf = wave_sum_u32(my_inf);
    __syncthreads();  // ds.n_inf is zero
    if ((tid & (kWave - 1)) == 0 && my_inf != 0) atomicAdd(&ds.n_inf, my_inf);
    const uint32_t kmax = block_max_u32_buf(lmax, ds.wave_u32);  // largest raw key; the barriers also publish the histogram
    if (kmax == kNegInfKey) return false;  // nothing above -inf: the draw is uniform over the row (radix path)
    const uint32_t n_inf = ds.n_inf;

    // ---- 2. compact the occupied keys, in descending order, into the list ---------------------------------
    // lane t owns the words [D_WORDS - 32 (t + 1), D_WORDS - 32 t) and walks them from the top
    const int block = D_WORDS / 32 - 1 - tid;
    // (the 128 bytes are read twice, 16 at a time, rather than held in 32 registers next to the row)
    auto chunk_of = [&](int c) {
        return *reinterpret_cast<const uint4 *>(&hist[(block << 5) | (((c ^ (block >> 1)) & 7) << 2)]);
    };
    uint32_t n_occ = 0, n_cnt = 0;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        const uint4 wv = chunk_of(c);
        const uint32_t q[4] = {wv.x, wv.y, wv.z, wv.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            n_occ += ((q[i] >> 16) != 0) + ((q[i] & 0xffffu) != 0);
            n_cnt += (q[i] >> 16) + (q[i] & 0xffffu);
        }
    }
    uint32_t occ_total, cnt_total;
    uint32_t at = block_excl_scan<uint32_t>(n_occ, ds.wave_u32, &occ_total);
    block_excl_scan<uint32_t>(n_cnt, ds.wave_u32, &cnt_total);
    // a 16-bit counter that overflowed loses 65,535 or 65,536 entries of the total; more occupied keys than
    // the list holds: leave the row to the radix path
    if (cnt_total + n_inf != uint32_t(vocab) || occ_total > uint32_t(D_LIST_CAP)) return false;
#pragma unroll
    for (int c = 7; c >= 0; --c) {
        const uint4 wv = chunk_of(c);
        const uint32_t q[4] = {wv.x, wv.y, wv.z, wv.w};
#pragma unroll
        for (int i = 3; i >= 0; --i) {
            const uint32_t key_hi = uint32_t(((block << 5) + c * 4 + i) * 2 + 1);
            if ((q[i] >> 16) != 0) list[at++] = (key_hi << 16) | (q[i] >> 16);
            if ((q[i] & 0xffffu) != 0) list[at++] = ((key_hi - 1) << 16) | (q[i] & 0xffffu);
        }
    }
    __syncthreads();

    // ---- 3. scaled key and mass, once per occupied key: lane t takes the entries [t * D_PER_THREAD, ...) -------
    // Several raw keys may scale to one value; such a run of entries is one tie group of the operator.
    uint16_t *const skl = reinterpret_cast<uint16_t *>(hist);  // scaled key of every list entry (the counts are spent)
    auto scaled = [&](uint32_t raw_key) -> uint32_t {
        if (!HAS_T) return raw_key;
        const uint32_t bits = (raw_key & 0x8000u) ? (raw_key & 0x7fffu) : (~raw_key & 0xffffu);
        return elem_key16<T, true>(bits, temp);
    };
    const uint32_t kmax_s = scaled(kmax);
    const float vmax = value_of_key16<T>(kmax_s);
    uint32_t ent[D_PER_THREAD], sk[D_PER_THREAD];
    uint64_t wgt[D_PER_THREAD];
    uint64_t m_local = 0;
    uint32_t c_local = 0;
#pragma unroll
    for (int e = 0; e < D_PER_THREAD; ++e) {
        const uint32_t i = uint32_t(tid) * D_PER_THREAD + e;
        ent[e] = i < occ_total ? list[i] : 0u;
        const uint32_t c = ent[e] & 0xffffu;
        sk[e] = scaled(ent[e] >> 16);
        wgt[e] = c ? weight_fix(sk[e] == kmax_s ? 0.0f : value_of_key16<T>(sk[e]) - vmax) : 0ull;
        m_local += wgt[e] * c;
        c_local += c;
        if (i < occ_total && !all_survive) skl[i] = uint16_t(sk[e]);
    }
    uint64_t z_all;
    uint32_t c_all;
    const uint64_t m_before = block_excl_scan<uint64_t>(m_local, ds.wave_u64, &z_all);
    const uint32_t c_before = block_excl_scan<uint32_t>(c_local, ds.wave_u32, &c_all);
    if (tid == 0) {
        ds.i_topk = occ_total - 1;
        ds.z_topk = z_all;
        ds.best_i = -1;
        ds.fail = 0;
    }
    __syncthreads();  // skl[] complete
    // last entry of the run (equal scaled keys) that contains entry i; a run longer than 64 entries (a huge
    // temperature folds many values together) is left to the radix path
    auto run_end = [&](uint32_t i) -> uint32_t {
        const uint32_t key = skl[i];
        uint32_t j = i;
        int guard = 0;
        while (j + 1 < occ_total && skl[j + 1] == key && guard < 64) { ++j; ++guard; }
        if (guard == 64) ds.fail = 1;
        return j;
    };

    // ---- the draw over the survivors in index order; mass(key) is the integer mass of an entry that survives
    //      entirely (0 otherwise), is_tie(key) marks the entries of a tie group of which only the first r_cut
    //      (in index order) survive, each with mass w_tie -------------------------------------------------------
    bool track_ties = false;
    uint32_t r_cut = 0xffffffffu;
    uint64_t w_tie = 0;
    uint32_t tie_hi = 0, tie_lo = 0;  // raw keys of the tie group that is cut

    // ---- no filter: every occupied key survives; its mass is found through the key's list index ---------------
    uint16_t *const idx16 = reinterpret_cast<uint16_t *>(hist);  // list index of every occupied raw key
    uint32_t kcut16 = 0, span = 0, first = 0;
    if (all_survive) {
        if (occ_total >= uint32_t(D_TABLE_CAP)) return false;  // the mass table holds 8 bytes per occupied key
        if (tid == 0) {  // the -inf entries look up a zero behind the last occupied key
            idx16[kNegInfKey] = uint16_t(occ_total);
            table[occ_total] = 0;
        }
#pragma unroll
        for (int e = 0; e < D_PER_THREAD; ++e) {
            const uint32_t i = uint32_t(tid) * D_PER_THREAD + e;
            if (i < occ_total) {
                idx16[ent[e] >> 16] = uint16_t(i);
                table[i] = wgt[e];  // every lane has read its list entries (barrier above)
            }
        }
        __syncthreads();
    } else {
    // ---- 4. top-k: the run that holds the top_k-th largest entry; everything down to its end survives ----------
    if (use_k) {
        if (c_before < uint32_t(top_k) && uint32_t(top_k) <= c_before + c_local) {
            uint32_t c_run = c_before;
#pragma unroll
            for (int e = 0; e < D_PER_THREAD; ++e) {
                const uint32_t c = ent[e] & 0xffffu;
                if (c_run < uint32_t(top_k) && uint32_t(top_k) <= c_run + c) ds.i_topk = run_end(uint32_t(tid) * D_PER_THREAD + e);
                c_run += c;
            }
        }
        __syncthreads();
        if (ds.i_topk / D_PER_THREAD == uint32_t(tid)) {  // mass of everything down to that entry
            uint64_t m_run = m_before;
#pragma unroll
            for (int e = 0; e < D_PER_THREAD; ++e) {
                m_run += wgt[e] * (ent[e] & 0xffffu);
                if (uint32_t(tid) * D_PER_THREAD + e == ds.i_topk) ds.z_topk = m_run;
            }
        }
        __syncthreads();
    }
    const uint32_t i_topk = ds.i_topk;
    const uint64_t z_topk = ds.z_topk;

    // ---- 5. top-p: the last run at or above i_topk whose first element has (mass before it) <= theta ----------
    uint32_t i_last = i_topk;       // last surviving list entry
    uint64_t z_kept = z_topk;
    if (use_p) {
        const uint64_t theta = floor_scale(top_p, z_topk);
        int best = -1;
        uint64_t m_run = m_before;
#pragma unroll
        for (int e = 0; e < D_PER_THREAD; ++e) {
            const uint32_t i = uint32_t(tid) * D_PER_THREAD + e;
            const uint32_t c = ent[e] & 0xffffu;
            const uint32_t prev = e > 0 ? sk[e - 1] : (i > 0 && i < occ_total ? uint32_t(skl[i - 1]) : 0xffffffffu);
            const bool start = i == 0 || prev != sk[e];
            if (c != 0 && start && i <= i_topk && m_run <= theta) best = int(i);
            m_run += wgt[e] * c;
        }
        if (best >= 0) atomicMax(&ds.best_i, best);
        __syncthreads();
        const uint32_t i_cut = uint32_t(ds.best_i);
        if (i_cut / D_PER_THREAD == uint32_t(tid)) {
            uint64_t m_run2 = m_before;
#pragma unroll
            for (int e = 0; e < D_PER_THREAD; ++e) {
                const uint32_t c = ent[e] & 0xffffu;
                if (uint32_t(tid) * D_PER_THREAD + e == i_cut) {
                    const uint32_t j_end = run_end(i_cut);
                    uint32_t n = 0;
                    for (uint32_t j = i_cut; j <= j_end; ++j) n += list[j] & 0xffffu;
                    ds.before_cut = m_run2;
                    ds.w_cut = wgt[e];
                    ds.n_cut = n;
                    ds.i_last = j_end;
                    ds.tie_hi = ent[e] >> 16;
                    ds.tie_lo = list[j_end] >> 16;
                }
                m_run2 += wgt[e] * c;
            }
        }
        __syncthreads();
        const uint64_t before = ds.before_cut, w_cut = ds.w_cut;
        const uint64_t n_cut = ds.n_cut;
        i_last = ds.i_last;
        uint64_t r = n_cut;
        if (w_cut > 0) {
            const uint64_t fit = (theta - before) / w_cut + 1;  // entries t with before + t * w <= theta
            r = fit < r ? fit : r;
        }
        z_kept = before + r * w_cut;
        if (r != n_cut) {  // the cut falls inside a tie group: only its first r entries, in index order, survive
            track_ties = true;
            r_cut = uint32_t(r);
            w_tie = w_cut;
            tie_hi = ds.tie_hi;
            tie_lo = ds.tie_lo;
        }
    }
    if (ds.fail) return false;
    // ---- 6. masses of the surviving raw keys into a table indexed by key - lowest surviving key ---------------
    if (tid == i_last / D_PER_THREAD) {
#pragma unroll
        for (int e = 0; e < D_PER_THREAD; ++e)
            if (uint32_t(tid) * D_PER_THREAD + e == i_last) ds.kcut16 = ent[e] >> 16;
    }
    __syncthreads();  // also: every lane is done reading the list
    kcut16 = ds.kcut16;
    span = kmax - kcut16 + 1;
    if (span >= uint32_t(D_TABLE_CAP)) return false;
    for (uint32_t i = tid; i <= span; i += S_THREADS) table[i] = 0;  // table[span] stays 0: the slot of every non-survivor
    __syncthreads();
#pragma unroll
    for (int e = 0; e < D_PER_THREAD; ++e) {
        const uint32_t i = uint32_t(tid) * D_PER_THREAD + e;
        if (i <= i_last && (ent[e] & 0xffffu) != 0) table[(ent[e] >> 16) - kcut16] = wgt[e];
    }
    __syncthreads();
    (void)z_kept;  // equals the total the draw computes from the table
    first = track_ties ? tie_hi + 1 : kcut16;  // lowest raw key whose entries all survive
    }  // filters
    // ---- 7. draw over the survivors in index order ------------------------------------------------------------
    auto mass = [&](uint32_t k) -> uint64_t {
        return all_survive ? table[idx16[k]] : table[k >= first ? k - kcut16 : span];
    };
    auto is_tie = [&](uint32_t k) { return track_ties && k >= tie_lo && k <= tie_hi; };
    // 7a. per wavefront: mass of the full survivors and number of tie-group entries of its share of the row
    {
        uint64_t m = 0;
        uint32_t t = 0;
        for_wave_vectors<T, false>(vp, n_here, 1.0f, [&](bool valid, bool, const uint32_t (&k)[8]) {
            if (valid) {
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    m += mass(k[j]);
                    t += is_tie(k[j]) ? 1u : 0u;
                }
            }
        });
        m = wave_sum_u64(m);
        t = wave_sum_u32(t);
        uint64_t mt = has_tail ? mass(tail_key) : 0ull;
        uint32_t tt = (has_tail && is_tie(tail_key)) ? 1u : 0u;
        if (wave == 0) {
            mt = wave_sum_u64(mt);
            tt = wave_sum_u32(tt);
        }
        if ((tid & (kWave - 1)) == 0) {
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
    // 7b. the segment (a wavefront's share, or the tail) that holds floor(u * Z)
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
    // 7c. inside the segment: the step, the lane, the entry (one wavefront works, the others wait at the barrier)
    if (seg == wave) {
        uint64_t cum = acc;
        uint32_t rank = ties_before;
        bool found = false;
        uint32_t hk[8] = {0, 0, 0, 0, 0, 0, 0, 0};  // this lane's keys in the step that holds tau
        bool hvalid = false;
        int hstep = 0, step = 0;
        uint64_t hcum = 0;
        uint32_t hrank = 0;
        for_wave_vectors<T, false>(vp, n_here, 1.0f, [&](bool valid, bool, const uint32_t (&k)[8]) {
            uint64_t m = 0;
            uint32_t t = 0;
            if (valid) {
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    m += mass(k[j]);
                    t += is_tie(k[j]) ? 1u : 0u;
                }
            }
            const uint64_t ms = wave_sum_u64(m);
            const uint32_t ts = wave_sum_u32(t);
            const uint32_t room = rank < r_cut ? r_cut - rank : 0u;
            const uint64_t total = ms + uint64_t(ts < room ? ts : room) * w_tie;
            if (!found && tau < cum + total) {  // wavefront-uniform
                found = true;
                hstep = step;
                hcum = cum;
                hrank = rank;
                hvalid = valid;
#pragma unroll
                for (int j = 0; j < 8; ++j) hk[j] = k[j];
            }
            cum += total;
            rank += ts;
            ++step;
        });
        // lanes of that step in order: tie ranks first, then masses
        uint32_t lt = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) lt += (hvalid && is_tie(hk[j])) ? 1u : 0u;
        uint32_t rk = hrank + wave_excl_scan<uint32_t>(lt);
        const uint32_t rk0 = rk;
        uint64_t lm = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j)
            if (hvalid) lm += is_tie(hk[j]) ? ((rk++ < r_cut) ? w_tie : 0ull) : mass(hk[j]);
        const uint64_t before = hcum + wave_excl_scan<uint64_t>(lm);
        if (before <= tau && tau < before + lm) {
            uint64_t c2 = before;
            uint32_t r2 = rk0;
            bool done = false;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint64_t wj = is_tie(hk[j]) ? ((r2++ < r_cut) ? w_tie : 0ull) : mass(hk[j]);
                c2 += wj;
                if (!done && c2 > tau) {
                    done = true;
                    ds.hit = (v0 + hstep * kWave + (tid & (kWave - 1))) * 8 + j;
                    ds.pick_w = wj;
                }
            }
        }
    } else if (seg == S_WAVES && wave == 0) {
        const bool tie = has_tail && is_tie(tail_key);
        const uint32_t rk = ties_before + wave_excl_scan<uint32_t>(tie ? 1u : 0u);
        const uint64_t wt = has_tail ? (tie ? (rk < r_cut ? w_tie : 0ull) : mass(tail_key)) : 0ull;
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
    return true;
}

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

template <typename T, bool DENSE>
__global__ __launch_bounds__(S_THREADS) void sample_rows(const typename T::raw_t *__restrict__ logits,
                                                         int vocab, int64_t row_stride, SampleParams prm, int vec,
                                                         int no_fast) {
    constexpr int EPV = T::kPerVec;
    constexpr int LEVELS = Round<T>::kLevels;
    unsigned char *const lds = lds_base<DENSE>();
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
    int64_t *__restrict__ out = prm.out_ids;
    float *lp_slot = prm.out_logprob != nullptr ? prm.out_logprob + row : nullptr;
    const bool has_t = temp != 1.0f;
    const bool use_k = top_k > 0 && top_k < vocab;
    const bool use_p = top_p < 1.0f;

    float u = uniforms[row];
    if (!(u >= 0.0f)) u = 0.0f;
    if (u >= 1.0f) u = __uint_as_float(0x3f7fffffu);

    if (use_k && top_k <= S_THREADS && !no_fast) {
        if (fast_topk<T>(sh, rp, vocab, vec, temp, has_t, top_k, use_p, top_p, u, out + row, lp_slot)) return;
        __syncthreads();
    } else if (!no_fast) {
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
            if (done) return;
            __syncthreads();
        }
        if constexpr (!DENSE && T::kBytes == 2) {
            if (!use_k && !use_p) {  // launched without the histogram's LDS: fp16, whose rows hold too many distinct values
                if (nofilter_resident<T>(sh.ds, rp, vocab, vec, temp, has_t, u, out + row, lp_slot)) return;
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
    uint64_t z_topk;
    block_excl_scan<uint64_t>(zpart, sh.wave_u64, &z_topk);
    __syncthreads();

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
}

__global__ __launch_bounds__(256) void mass_fixed_kernel(const float *__restrict__ d, int64_t n, uint64_t *__restrict__ out) {
    const int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) out[i] = weight_fix(d[i]);
}

// KA_SAMPLE_RADIX_ONLY=1 switches the top-k fast path off (the tests use it to run both paths on every case).
inline bool force_radix_path() {
    const char *e = getenv("KA_SAMPLE_RADIX_ONLY");
    return e != nullptr && e[0] == '1';
}

template <typename T>
int launch(const void *logits, int64_t batch, int64_t vocab, int64_t row_stride, const SampleParams &prm,
           void *workspace, size_t workspace_bytes, void *hip_stream) {
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
    const bool no_fast = force_radix_path();
    // The dense-histogram path needs 157 KB of LDS (one workgroup per CU).  It serves top-p without top-k and
    // top_k > 1024 on 16-bit rows that fit in registers; with per-row parameters any row may need it.
    bool dense = false;
    if (T::kBytes == 2 && aligned && !no_fast && vocab / 8 <= RES_VECS * S_THREADS) {
        const bool per_row = prm.top_k_rows != nullptr || prm.top_p_rows != nullptr;
        const bool k_on = prm.top_k > 0 && prm.top_k < vocab;
        // (no filter at all: the histogram path for bf16; an fp16 row has too many distinct values for its list and
        //  takes the register-resident no-filter path of the small-LDS kernel)
        const bool no_filter = !k_on && !(prm.top_p < 1.0f);
        dense = per_row || (k_on && prm.top_k > S_THREADS) || (!k_on && !no_filter) ||
                (no_filter && T::kDtype == KA_DTYPE_BF16);
    }
    hipStream_t stream = static_cast<hipStream_t>(hip_stream);
    const typename T::raw_t *lp = static_cast<const typename T::raw_t *>(logits);
    if constexpr (T::kBytes == 2) {
      if (dense) {
        const hipError_t rc = hipFuncSetAttribute(reinterpret_cast<const void *>(sample_rows<T, true>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, int(DENSE_LDS_BYTES));
        if (rc != hipSuccess) return check_hip(rc, "sample: reserving LDS for the dense-histogram path");
        hipLaunchKernelGGL((sample_rows<T, true>), dim3(unsigned(batch)), dim3(S_THREADS), DENSE_LDS_BYTES, stream, lp,
                           int(vocab), row_stride, prm, aligned ? 1 : 0, 0);
        return check_hip(hipGetLastError(), "sample launch");
      }
    }
    hipLaunchKernelGGL((sample_rows<T, false>), dim3(unsigned(batch)), dim3(S_THREADS), 0, stream, lp, int(vocab),
                       row_stride, prm, aligned ? 1 : 0, no_fast ? 1 : 0);
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
                     const SampleParams &prm, void *workspace, size_t workspace_bytes, void *hip_stream) {
    switch (dtype) {
        case KA_DTYPE_BF16: return launch<Bf16>(logits, batch, vocab, row_stride, prm, workspace, workspace_bytes, hip_stream);
        case KA_DTYPE_F16: return launch<F16>(logits, batch, vocab, row_stride, prm, workspace, workspace_bytes, hip_stream);
        case KA_DTYPE_F32: return launch<F32>(logits, batch, vocab, row_stride, prm, workspace, workspace_bytes, hip_stream);
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
                           int64_t *out_ids, float *out_logprob, void *workspace, size_t workspace_bytes,
                           void *hip_stream) {
    ka::SampleParams p = ka::scalar_params(temperature, top_k, top_p, uniforms, out_ids);
    p.temperature_rows = temperature_rows;
    p.top_k_rows = top_k_rows;
    p.top_p_rows = top_p_rows;
    p.out_logprob = out_logprob;
    return ka::launch_ex(dtype, logits, batch, vocab, row_stride, p, workspace, workspace_bytes, hip_stream);
}

// Shared pieces of the sampling kernels: order-preserving keys, the integer mass function, exact floor(s * z),
// temperature rounding, radix level layout, LDS state, block-wide primitives and row traversal.
#ifndef KA_SAMPLING_COMMON_H
#define KA_SAMPLING_COMMON_H

#include <type_traits>

#include "ka_common.h"

namespace ka {
namespace {

// Phase stamps for timing experiments (block 0, thread 0 writes the shader clock at named points).
#ifdef KA_SAMPLE_STAMPS
__device__ unsigned long long ka_dbg_stamps[16 * 16 + 32];  // [wavefront][point], then 32 free slots
#define KA_STAMP(i_) do { if (blockIdx.x == 0 && (threadIdx.x & 63) == 0) ka_dbg_stamps[(threadIdx.x >> 6) * 16 + (i_)] = __builtin_readcyclecounter(); } while (0)
#define KA_DBG_SET(i_, v_) do { ka_dbg_stamps[256 + (i_)] = (unsigned long long)(v_); } while (0)
#else
#define KA_STAMP(i_) do { } while (0)
#define KA_DBG_SET(i_, v_) do { } while (0)
#endif

// Threads of a workgroup (one row).  1024 is the ordinary build.  A second build of the top-k kernel with 512 lets two
// workgroups share a CU, so that one row's selection runs under the other row's read; it is launched for batches of more
// rows than the device has CUs.  Every integer decision is the same function of the row in both.
#ifndef KA_SAMPLING_THREADS
#define KA_SAMPLING_THREADS 1024
#endif
constexpr int S_THREADS = KA_SAMPLING_THREADS;
static_assert(S_THREADS == 1024 || S_THREADS == 512, "the sampling kernels are written for 1024 or 512 threads");
constexpr int S_WAVES = S_THREADS / kWave;
constexpr int BINS = 2048;
constexpr int BINS_PER_THREAD = BINS / S_THREADS;  // of a histogram that the block scans in one step
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
    uint32_t n_ge, surv_overflow;    // dense path: entries at or above the lowest surviving key; a wavefront's survivor list overflowed
    uint32_t seg_cnt[S_WAVES];       // ... survivors listed by each wavefront
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
    uint32_t n_cand, n_vec, cand_kmax, pick_a, pick_b;
    uint64_t pick_z;
    DenseScalars ds;  // scalars of the resident no-filter path
};

// Cross-lane moves inside a row of sixteen lanes (DPP: no LDS traffic): lane ^ 1, lane ^ 2, 7 - lane inside each
// half row, and 15 - lane.  Applied in this order, a sum (or maximum) over 2, 4, 8, 16 neighbouring lanes builds up.
__device__ __forceinline__ uint32_t dpp_xor1(uint32_t v) { return uint32_t(__builtin_amdgcn_update_dpp(0, int(v), 0xB1, 0xf, 0xf, false)); }
__device__ __forceinline__ uint32_t dpp_xor2(uint32_t v) { return uint32_t(__builtin_amdgcn_update_dpp(0, int(v), 0x4E, 0xf, 0xf, false)); }
__device__ __forceinline__ uint32_t dpp_row_mirror(uint32_t v) { return uint32_t(__builtin_amdgcn_update_dpp(0, int(v), 0x140, 0xf, 0xf, false)); }
__device__ __forceinline__ uint32_t dpp_half_mirror(uint32_t v) { return uint32_t(__builtin_amdgcn_update_dpp(0, int(v), 0x141, 0xf, 0xf, false)); }

// Inclusive prefix sum of one 64-bit value per lane over the wavefront, by DPP row shifts and row broadcasts.
// One step: lanes outside ROW_MASK, and lanes whose source lies outside the row, add 0.
template <int CTRL, int ROW_MASK> __device__ __forceinline__ uint64_t scan_step_u64(uint64_t v) {
    const uint32_t lo = uint32_t(__builtin_amdgcn_update_dpp(0, int(uint32_t(v)), CTRL, ROW_MASK, 0xf, true));
    const uint32_t hi = uint32_t(__builtin_amdgcn_update_dpp(0, int(uint32_t(v >> 32)), CTRL, ROW_MASK, 0xf, true));
    return v + ((uint64_t(hi) << 32) | lo);
}
__device__ __forceinline__ uint64_t wave_incl_scan_u64(uint64_t v) {
    v = scan_step_u64<0x111, 0xf>(v);  // row_shr:1
    v = scan_step_u64<0x112, 0xf>(v);  // row_shr:2
    v = scan_step_u64<0x114, 0xf>(v);  // row_shr:4
    v = scan_step_u64<0x118, 0xf>(v);  // row_shr:8
    v = scan_step_u64<0x142, 0xa>(v);  // row_bcast:15 -> rows 1 and 3
    v = scan_step_u64<0x143, 0xc>(v);  // row_bcast:31 -> rows 2 and 3
    return v;
}

template <int CTRL, int ROW_MASK> __device__ __forceinline__ uint32_t scan_step_u32(uint32_t v) {
    return v + uint32_t(__builtin_amdgcn_update_dpp(0, int(v), CTRL, ROW_MASK, 0xf, true));
}
__device__ __forceinline__ uint32_t wave_incl_scan_u32(uint32_t v) {
    v = scan_step_u32<0x111, 0xf>(v);
    v = scan_step_u32<0x112, 0xf>(v);
    v = scan_step_u32<0x114, 0xf>(v);
    v = scan_step_u32<0x118, 0xf>(v);
    v = scan_step_u32<0x142, 0xa>(v);
    v = scan_step_u32<0x143, 0xc>(v);
    return v;
}
__device__ __forceinline__ uint32_t wave_incl_scan(uint32_t v) { return wave_incl_scan_u32(v); }
__device__ __forceinline__ uint64_t wave_incl_scan(uint64_t v) { return wave_incl_scan_u64(v); }

template <typename V> __device__ __forceinline__ V shfl_up_v(V v, int off) { return __shfl_up(v, off, kWave); }

// Exclusive prefix sum over the block in thread order; *total = block sum.  Contains barriers; every thread of the
// block must call it (the wavefront-level part moves data by DPP, which needs all 64 lanes active).
template <typename V>
__device__ __forceinline__ V block_excl_scan(V v, V *wave_buf, V *total) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const V inc = wave_incl_scan(v);
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
    // thread t owns the bins BINS_PER_THREAD * t + j counted from the top
    uint32_t c[BINS_PER_THREAD], mine = 0;
#pragma unroll
    for (int j = 0; j < BINS_PER_THREAD; ++j) {
        const int rb = BINS_PER_THREAD * tid + j;
        c[j] = rb < int(nb) ? sh.h.cnt[nb - 1 - rb] : 0u;
        mine += c[j];
    }
    uint32_t total;
    uint32_t run = block_excl_scan<uint32_t>(mine, sh.wave_u32, &total);
#pragma unroll
    for (int j = 0; j < BINS_PER_THREAD; ++j) {
        if (run < rank && rank <= run + c[j]) {
            sh.sel_digit = nb - 1 - uint32_t(BINS_PER_THREAD * tid + j); sh.sel_above = run; sh.sel_count = c[j];
        }
        run += c[j];
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
// Log-sum-exp of the raw row, taken along by the sampling kernel when the caller wants the drawn token's
// log-probability under the unfiltered softmax (what the logprob operator returns for it).  A lane folds its
// elements online in fp32 (base-2 exponentials relative to a running maximum), the lanes of a wavefront are folded by
// a fixed butterfly, the wavefronts in wavefront order: the value depends on the row and on the route its sampling
// takes, not on the batch.
// ---------------------------------------------------------------------------
constexpr float kLseLog2e = 1.44269504088896340736f;
constexpr float kLseFloor = -1.0e30f;  // running maxima start here: (old max - new max) is never inf - inf

// The fold is defined on 1024 lanes: lane t takes the vectors t, t + 1024, ... of the row.  A block of 512 threads lets
// thread t stand in for the lanes t and t + 512 with an accumulator each, so both builds return the same bits.
constexpr int LSE_LANES = 1024;
constexpr int LSE_WAVES = LSE_LANES / kWave;
constexpr int LSE_PER_THREAD = LSE_LANES / S_THREADS;

struct PolicyLse {  // in LDS
    float wave_ml2[LSE_WAVES];  // maximum * log2(e) of the elements of each wavefront of the 1024-lane order
    float wave_s[LSE_WAVES];    // sum of 2^(x * log2(e) - wave_ml2)
    // log-probability of element `hit` of the row (thread 0, after a barrier behind to_block)
    template <typename T> __device__ __forceinline__ float finish(const typename T::raw_t *rp, int64_t hit, int vocab) const {
        if (hit < 0 || hit >= vocab) return __builtin_nanf("");
        float big = wave_ml2[0];
#pragma unroll
        for (int w = 1; w < LSE_WAVES; ++w) big = fmaxf(big, wave_ml2[w]);
        float total = 0.0f;
#pragma unroll
        for (int w = 0; w < LSE_WAVES; ++w) total += wave_s[w] * fast_exp2(wave_ml2[w] - big);
        const double lse = (double(big) + log2(double(total))) * 0.693147180559945309417232;
        return float(double(T::widen(rp[hit])) - lse);
    }
};

struct LaneLse {
    float m = kLseFloor, ml2 = kLseFloor * kLseLog2e, s = 0.0f;
    // Contraction is off in these functions: fused into an FMA against the fresh product, (ml2 - mn * log2e) would return
    // the rounding residue of a 1e30-sized product instead of 0 while the maximum still sits at the floor, and 2^residue
    // overflows.
    __device__ __forceinline__ void add(float x) {
#pragma clang fp contract(off)
        const float mn = fmaxf(m, x);
        const float ml2n = mn * kLseLog2e;
        s = fmaf(s, fast_exp2(ml2 - ml2n), fast_exp2(fmaf(x, kLseLog2e, -ml2n)));
        m = mn;
        ml2 = ml2n;
    }
    // N elements whose maximum vm is known already: one rescale for all of them
    template <int N> __device__ __forceinline__ void add_vector(const float (&x)[N], float vm) {
#pragma clang fp contract(off)
        const float mn = fmaxf(m, vm);
        const float ml2n = mn * kLseLog2e;
        float e = 0.0f;
#pragma unroll
        for (int j = 0; j < N; ++j) e += fast_exp2(fmaf(x[j], kLseLog2e, -ml2n));
        s = fmaf(s, fast_exp2(ml2 - ml2n), e);
        m = mn;
        ml2 = ml2n;
    }
    // every thread of the block calls this; a barrier must follow before PolicyLse::finish.  `stand_in`: which of the
    // thread's lanes of the 1024-lane order this accumulator belongs to (lane threadIdx.x + stand_in * S_THREADS).
    __device__ __forceinline__ void to_block(PolicyLse &out, int stand_in = 0) const {
        const float wm = wave_max(ml2);
        const float ws = wave_sum(s * fast_exp2(ml2 - wm));
        if ((threadIdx.x & (kWave - 1)) == 0) {
            out.wave_ml2[threadIdx.x / kWave + stand_in * S_WAVES] = wm;
            out.wave_s[threadIdx.x / kWave + stand_in * S_WAVES] = ws;
        }
    }
};

// The accumulators of one thread: one per lane of the 1024-lane order it stands in for.
struct ThreadLse {
    LaneLse lane[LSE_PER_THREAD];
    __device__ __forceinline__ void to_block(PolicyLse &out) const {
#pragma unroll
        for (int e = 0; e < LSE_PER_THREAD; ++e) lane[e].to_block(out, e);
    }
};

// Largest element of a 16-byte vector.
template <typename T> __device__ __forceinline__ float vector_max(const uint4 &q) {
    const typename T::raw_t *e = reinterpret_cast<const typename T::raw_t *>(&q);
    float vm = T::widen(e[0]);
#pragma unroll
    for (int j = 1; j < T::kPerVec; ++j) vm = fmaxf(vm, T::widen(e[j]));
    return vm;
}

// Log-sum-exp partials of a whole row by the block, in the order the short top-k route folds a row while it reads it:
// lane t of the 1024-lane order takes the vectors t, t + 1024, ... (one rescale per vector), then element t of the ragged
// tail; an unaligned row goes element by element (t, t + 1024, ...).  The value is a function of the row alone.
template <typename T>
__device__ __forceinline__ void row_lse_to_block(const typename T::raw_t *rp, int vocab, bool vec, PolicyLse &out) {
    constexpr int EPV = T::kPerVec;
    ThreadLse acc;
#pragma unroll
    for (int e = 0; e < LSE_PER_THREAD; ++e) {
        const int lane = int(threadIdx.x) + e * S_THREADS;
        if (vec) {
            const uint4 *vp = reinterpret_cast<const uint4 *>(rp);
            const int nvec = vocab / EPV;
            constexpr int U = 4;  // loads in flight; the vectors are folded in their order
            auto fold = [&](const uint4 &q) {
                float x[EPV];
                T::unpack(q, x);
                acc.lane[e].add_vector(x, vector_max<T>(q));
            };
            int v = lane;
            for (; v + (U - 1) * LSE_LANES < nvec; v += U * LSE_LANES) {
                uint4 q[U];
#pragma unroll
                for (int u = 0; u < U; ++u) q[u] = vp[v + u * LSE_LANES];
#pragma unroll
                for (int u = 0; u < U; ++u) fold(q[u]);
            }
            for (; v < nvec; v += LSE_LANES) fold(vp[v]);
            const int i = nvec * EPV + lane;
            if (i < vocab) acc.lane[e].add(T::widen(rp[i]));
        } else {
            for (int i = lane; i < vocab; i += LSE_LANES) acc.lane[e].add(T::widen(rp[i]));
        }
    }
    acc.to_block(out);
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

}  // namespace
}  // namespace ka

#endif  // KA_SAMPLING_COMMON_H

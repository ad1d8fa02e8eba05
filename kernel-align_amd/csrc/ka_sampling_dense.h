// Paths of the sampling kernel for 16-bit dtypes: the register-resident no-filter path and the dense-histogram path.
#ifndef KA_SAMPLING_DENSE_H
#define KA_SAMPLING_DENSE_H

#include "ka_sampling_common.h"

namespace ka {
namespace {

// ---------------------------------------------------------------------------
// Paths for 16-bit dtypes (bf16, fp16), 16-byte aligned rows (the register-resident no-filter path: at most
// 131,072 entries; the dense path streams the row and takes any length).
// Since a 16-bit dtype has only 65,536 values, an entry's integer mass is a function of its 16-bit key.
//
//   no filter   : the row is read once into registers (16 x uint4 per lane, a contiguous run of entries per
//                 lane) and every entry is replaced by the key of its scaled value; one pass evaluates every
//                 entry's mass, one block-wide prefix sum of the lane totals finds the lane that holds the
//                 draw, which then finds the vector and the entry.
//   dense path  : (no filter on bf16 rows, top-p without top-k, or top_k > 1024) a count histogram over all 65,536 raw keys in LDS
//                 (16-bit counters, two per word) is filled by one streaming pass and compacted into a list
//                 of the occupied keys in descending order; temperature and masses are applied once per
//                 occupied key (a few thousand instead of 128 K; runs of keys that scale to one value form
//                 one tie group); prefix sums over the list give the top-k key, Z, the top-p cut and the
//                 surviving mass; the masses of the surviving keys go into a table indexed by
//                 key - lowest surviving key, and the draw streams the row once more (from L2 / MALL) for the
//                 mass of every wavefront's share, then re-reads the share that holds the target, one 64-vector
//                 step per wavefront, to find the step, the lane and the entry.
// Both return false (having written no output) when a row does not fit (a counter overflow, too many occupied
// keys, survivors spanning too many keys, a temperature that folds more than 64 values into one); the radix
// path then runs.  All integer decisions are the same function of the row as in the radix path.
// ---------------------------------------------------------------------------
constexpr int RES_VECS = 16;
constexpr int D_WORDS = 32768;              // 65,536 16-bit counters
constexpr int D_LIST_CAP = 7168;            // occupied keys the list can hold (4 B each)
constexpr int D_TABLE_CAP = D_LIST_CAP / 2; // keys spanned by the survivors (8 B each, same LDS region)
constexpr int D_PER_THREAD = D_LIST_CAP / S_THREADS;  // list entries per thread
constexpr int D_SURV_SEG = 512;             // survivors per wavefront the list-based draw of the filtered modes takes (12 B each)
constexpr int D_SURV_DEFER = 2048;          // ... and in all (more survivors: the streaming draw is faster)
static_assert(size_t(S_WAVES + 1) * D_SURV_SEG * 12 <= size_t(D_WORDS) * 4, "the survivor lists live in the histogram's memory");

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

// Sums over the 64 lanes of a wavefront (all lanes active), the total in every lane: a DPP prefix sum, then lane 63.
__device__ __forceinline__ uint64_t wave_sum_u64(uint64_t v) {
    const uint64_t inc = wave_incl_scan_u64(v);
    return (uint64_t(uint32_t(__builtin_amdgcn_readlane(int(uint32_t(inc >> 32)), kWave - 1))) << 32) |
           uint32_t(__builtin_amdgcn_readlane(int(uint32_t(inc)), kWave - 1));
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

typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
typedef short i16x2 __attribute__((ext_vector_type(2)));

// Key j (0..7) of a vector whose keys are packed two per dword (entry 2c in the low half of dword c).
__device__ __forceinline__ uint32_t key_at(const uint32_t (&kk)[4], int j) {
    return (j & 1) ? kk[j >> 1] >> 16 : kk[j >> 1] & 0xffffu;
}

// The eight 16-bit keys of one 16-byte vector, two per dword.  Returns true if none of the values is a zero, an
// infinity or a NaN (only looked for without a temperature): such a vector is converted with packed 16-bit
// instructions, three per two keys, and no selects.
template <typename T, bool HAS_T>
__device__ __forceinline__ bool vector_keys(const uint4 &q, float temp, uint32_t (&kk)[4]) {
    const uint32_t in[4] = {q.x, q.y, q.z, q.w};
    bool plain = false;
    if constexpr (!HAS_T) {
        // magnitude - 1 (wrapping in 16 bits) is 0xffff for a zero and at least kInf - 1 for an infinity or a NaN
        constexpr uint32_t kInf = T::kDtype == KA_DTYPE_BF16 ? 0x7f80u : 0x7c00u;
        u16x2 worst = {0, 0};
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const u16x2 mag = __builtin_bit_cast(u16x2, in[c] & 0x7fff7fffu);
            worst = __builtin_elementwise_max(worst, mag - u16x2{1, 1});
        }
        const uint32_t w = __builtin_bit_cast(uint32_t, worst);
        const uint32_t m = (w & 0xffffu) > (w >> 16) ? (w & 0xffffu) : (w >> 16);
        plain = m < kInf - 1u;
    }
    if (plain) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint32_t neg = __builtin_bit_cast(uint32_t, __builtin_bit_cast(i16x2, in[c]) >> 15);  // 0xffff in each negative half
            kk[c] = in[c] ^ (neg | 0x80008000u);
        }
    } else {
#pragma unroll
        for (int c = 0; c < 4; ++c)
            kk[c] = elem_key16<T, HAS_T>(in[c] & 0xffffu, temp) | (elem_key16<T, HAS_T>(in[c] >> 16, temp) << 16);
    }
    return plain;
}

// Walks the vectors of this wavefront's share of the row: wavefront w owns the vectors [w * vpw, (w + 1) * vpw)
// (a contiguous sixteenth of the row, so index order is (wavefront, step, lane, entry)), lane l takes the
// vectors l, l + 64, ... of that share: every load instruction covers 1 KB of consecutive memory.  Calls
// f(valid, plain, keys) once per step with the eight 16-bit keys of the lane's vector, packed two per dword
// (plain: see vector_keys);
// the trip count is the same for all lanes, so f may contain wavefront-wide exchanges.  Four loads are in
// flight per lane.
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
                uint32_t kk[4];
                const bool plain = vector_keys<T, HAS_T>(q[s], temp, kk);
                f(i0 + s * kWave + lane < n_here, plain, kk);
            }
        }
    }
}

__device__ __forceinline__ uint32_t wave_sum_u32(uint32_t v) {
    return uint32_t(__builtin_amdgcn_readlane(int(wave_incl_scan_u32(v)), kWave - 1));
}
// Exclusive prefix sums over the 64 lanes of a wavefront (all lanes active).
template <typename V> __device__ __forceinline__ V wave_excl_scan(V v) { return wave_incl_scan(v) - v; }

template <typename T, bool HAS_T, bool ALL_SURVIVE>
__device__ __forceinline__ bool dense_stream(unsigned char *lds, const typename T::raw_t *rp, int vocab, bool vec,
                                             float temp, bool use_k, int top_k, bool use_p, float top_p, float u,
                                             int64_t *out_slot, float *lp_slot) {
    if (!vec || T::kBytes != 2) return false;  // rows of any length: nothing of the row is kept
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
    u16x2 lmax2 = {0, 0};
    unsigned char *const hist_bytes = reinterpret_cast<unsigned char *>(hist);
    for_wave_vectors<T, false>(vp, n_here, 1.0f, [&](bool valid, bool plain, const uint32_t (&kk)[4]) {
        if (valid && plain) {
            // two keys per dword all the way: histogram word of a key = key >> 1, swizzled as in hist_slot(); its
            // counter is the low half for an even key, the high half for an odd one
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                lmax2 = __builtin_elementwise_max(lmax2, __builtin_bit_cast(u16x2, kk[c]));
                const uint32_t w2 = (kk[c] >> 1) & 0x7fff7fffu;
                const uint32_t slot2 = w2 ^ ((w2 >> 4) & 0x001c001cu);
                atomicAdd(reinterpret_cast<uint32_t *>(hist_bytes + ((slot2 << 2) & 0x3fffcu)), (kk[c] & 1u) * 0xffffu + 1u);
                atomicAdd(reinterpret_cast<uint32_t *>(hist_bytes + ((slot2 >> 14) & 0x3fffcu)),
                          ((kk[c] >> 16) & 1u) * 0xffffu + 1u);
            }
        } else if (valid) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint32_t k = key_at(kk, j);
                if (k == kNegInfKey) ++my_inf;
                else atomicAdd(&hist[hist_slot(k >> 1)], (k & 1) ? 0x10000u : 1u);
                lmax = k > lmax ? k : lmax;
            }
        }
    });
    {
        const uint32_t m2 = __builtin_bit_cast(uint32_t, lmax2);
        lmax = (m2 & 0xffffu) > lmax ? (m2 & 0xffffu) : lmax;
        lmax = (m2 >> 16) > lmax ? (m2 >> 16) : lmax;
    }
    if (has_tail && tail_key != kNegInfKey) atomicAdd(&hist[hist_slot(tail_key >> 1)], (tail_key & 1) ? 0x10000u : 1u);
    my_inf = wave_sum_u32(my_inf);
    __syncthreads();  // ds.n_inf is zero
    if ((tid & (kWave - 1)) == 0 && my_inf != 0) atomicAdd(&ds.n_inf, my_inf);
    const uint32_t kmax = block_max_u32_buf(lmax, ds.wave_u32);  // largest raw key; the barriers also publish the histogram
    KA_STAMP(1);   // histogram pass
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

    KA_STAMP(2);   // occupied keys compacted
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
    KA_STAMP(3);   // masses of the occupied keys
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
        uint32_t c_run = c_before;
#pragma unroll
        for (int e = 0; e < D_PER_THREAD; ++e) {
            c_run += ent[e] & 0xffffu;
            if (uint32_t(tid) * D_PER_THREAD + e == i_last) {
                ds.kcut16 = ent[e] >> 16;
                ds.n_ge = c_run;  // entries of the row at or above the lowest surviving key
            }
        }
    }
    if (tid == 0) ds.surv_overflow = 0;
    if (tid < S_WAVES) ds.seg_cnt[tid] = 0;
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
    auto is_tie = [&](uint32_t k) { return track_ties && k >= tie_lo && k <= tie_hi; };
    KA_STAMP(4);   // filters and mass table
    // ---- 7'. the survivors are few (a top-p nucleus of a peaked distribution, a top-k of a few thousand) and all
    //          positive: list them and draw on the list instead of streaming the masses of the whole row -------------
    // The row is read once more, but a vector only costs a packed signed maximum of its raw bits and a compare with the
    // lowest surviving value (positive values order as their bit patterns).  The few vectors that hold a survivor are
    // read again from L2, one per lane and turn, and their survivors go to a list per wavefront (the wavefront's share
    // of the row is a contiguous sixteenth) with their masses.  The per-wavefront totals pick the share that holds
    // floor(u * Z) exactly as in 7b; the block ranks that share's survivors by index, and one wavefront walks them with
    // prefix sums.
    if constexpr (!ALL_SURVIVE) {
        const int lane = tid & (kWave - 1);
        if (ds.n_ge <= uint32_t(D_SURV_DEFER) && kcut16 > 0x8000u && vpw <= 32 * kWave) {  // the same for the whole block
            uint32_t *const s_idx = hist;                                                   // [S_WAVES][D_SURV_SEG], bit 31: tie-group entry
            uint64_t *const s_w = reinterpret_cast<uint64_t *>(hist + S_WAVES * D_SURV_SEG);  // the histogram's memory is free by now
            uint32_t *const o_idx = hist + 3 * S_WAVES * D_SURV_SEG;                         // the chosen share, in index order
            uint64_t *const o_w = reinterpret_cast<uint64_t *>(o_idx + D_SURV_SEG);
            // which of the lane's vectors hold a value at or above the cut (bit s: vector s * 64 + lane of the share)
            const int cut_raw = int(kcut16 & 0x7fffu);
            uint32_t hits = 0;
#pragma unroll 1
            for (int i0 = 0; i0 < n_here; i0 += 4 * kWave) {
                uint4 q[4];
#pragma unroll
                for (int sq = 0; sq < 4; ++sq) {
                    const int idx = i0 + sq * kWave + lane;
                    q[sq] = idx < n_here ? vp[idx] : make_uint4(0x80008000u, 0x80008000u, 0x80008000u, 0x80008000u);
                }
#pragma unroll
                for (int sq = 0; sq < 4; ++sq) {
                    i16x2 top = __builtin_elementwise_max(__builtin_bit_cast(i16x2, q[sq].x), __builtin_bit_cast(i16x2, q[sq].y));
                    top = __builtin_elementwise_max(top, __builtin_elementwise_max(__builtin_bit_cast(i16x2, q[sq].z),
                                                                                  __builtin_bit_cast(i16x2, q[sq].w)));
                    const int best = top.x > top.y ? int(top.x) : int(top.y);  // a NaN pattern passes: sorted out below
                    hits |= (best >= cut_raw ? 1u : 0u) << (i0 / kWave + sq);
                }
            }
            uint64_t m_lane = 0;
            uint32_t t_lane = 0;
            bool overflow = false;
            while (__any(hits != 0)) {
                if (hits != 0) {
                    const int sbit = __ffs(hits) - 1;
                    hits &= hits - 1;
                    const int idx = sbit * kWave + lane;
                    uint32_t kk[4];
                    vector_keys<T, false>(vp[idx], 1.0f, kk);
                    uint32_t smask = 0;
#pragma unroll
                    for (int j = 0; j < 8; ++j) smask |= (key_at(kk, j) >= kcut16 ? 1u : 0u) << j;
                    if (smask != 0) {
                        const uint32_t cnt = uint32_t(__popc(smask));
                        uint32_t pos = atomicAdd(&ds.seg_cnt[wave], cnt);
                        if (pos + cnt <= uint32_t(D_SURV_SEG)) {
                            pos += uint32_t(wave) * D_SURV_SEG;
#pragma unroll
                            for (int j = 0; j < 8; ++j) {
                                if ((smask >> j) & 1u) {
                                    const uint32_t key = key_at(kk, j);
                                    const bool tie = is_tie(key);
                                    const uint64_t wv = tie ? 0ull : table[key >= first ? key - kcut16 : span];
                                    s_idx[pos] = uint32_t((v0 + idx) * 8 + j) | (tie ? 0x80000000u : 0u);
                                    s_w[pos] = wv;
                                    ++pos;
                                    m_lane += wv;
                                    t_lane += tie ? 1u : 0u;
                                }
                            }
                        } else {
                            overflow = true;
                        }
                    }
                }
            }
            const uint64_t m = wave_sum_u64(m_lane);
            const uint32_t t = wave_sum_u32(t_lane);
            const bool tail_tie = has_tail && is_tie(tail_key);
            uint64_t mt = (has_tail && !tail_tie && tail_key >= kcut16) ? table[tail_key >= first ? tail_key - kcut16 : span] : 0ull;
            uint32_t tt = tail_tie ? 1u : 0u;
            if (wave == 0) {
                mt = wave_sum_u64(mt);
                tt = wave_sum_u32(tt);
            }
            if (__any(overflow) && lane == 0) ds.surv_overflow = 1;
            if (lane == 0) {
                ds.seg_mass[wave] = m;
                ds.seg_ties[wave] = t;
                if (wave == 0) {
                    ds.seg_mass[S_WAVES] = mt;
                    ds.seg_ties[S_WAVES] = tt;
                }
            }
            __syncthreads();
            KA_STAMP(11);
            if (!ds.surv_overflow) {  // (else a share holds more survivors than its list: the streaming draw below runs)
                // the share (or the ragged tail) that holds floor(u * Z): as in 7b below
                uint64_t z = 0;
                {
                    uint32_t seen = 0;
#pragma unroll
                    for (int g = 0; g <= S_WAVES; ++g) {
                        const uint32_t tg = ds.seg_ties[g];
                        const uint32_t room = seen < r_cut ? r_cut - seen : 0u;
                        z += ds.seg_mass[g] + uint64_t(tg < room ? tg : room) * w_tie;
                        seen += tg;
                    }
                }
                const uint64_t tau = floor_scale(u, z);
                uint64_t acc = 0;
                uint32_t ties_before = 0;
                int seg = -1;
                {
                    uint32_t seen = 0;
#pragma unroll
                    for (int g = 0; g <= S_WAVES; ++g) {
                        const uint32_t tg = ds.seg_ties[g];
                        const uint32_t room = seen < r_cut ? r_cut - seen : 0u;
                        const uint64_t mg = ds.seg_mass[g] + uint64_t(tg < room ? tg : room) * w_tie;
                        if (seg < 0 && tau < acc + mg) { seg = g; ties_before = seen; }
                        if (seg < 0) acc += mg;
                        seen += tg;
                    }
                }
                const uint32_t n = (seg >= 0 && seg < S_WAVES) ? ds.seg_cnt[seg] : 0u;
                if (n > 0) {
                    // the share's survivors were listed in no particular order: file them by index
                    const uint32_t *const u_idx = s_idx + uint32_t(seg) * D_SURV_SEG;
                    const uint64_t *const u_w = s_w + uint32_t(seg) * D_SURV_SEG;
                    auto file_by_index = [&](auto parts_c) {
                        constexpr uint32_t PARTS = decltype(parts_c)::value;
                        const uint32_t c = uint32_t(tid) / PARTS, part = uint32_t(tid) % PARTS;
                        uint32_t mine = 0, before = 0;
                        if (c < n) {
                            mine = u_idx[c];
                            const uint4 *i4 = reinterpret_cast<const uint4 *>(u_idx);
                            for (uint32_t g4 = part; g4 * 4 < n; g4 += PARTS) {
                                const uint4 iq = i4[g4];
                                const uint32_t ik[4] = {iq.x, iq.y, iq.z, iq.w};
#pragma unroll
                                for (int e = 0; e < 4; ++e)
                                    before += (g4 * 4 + e < n && (ik[e] & 0x7fffffffu) < (mine & 0x7fffffffu)) ? 1u : 0u;
                            }
                        }
                        before += dpp_xor1(before);
                        if (PARTS >= 4) before += dpp_xor2(before);
                        if (PARTS >= 8) before += dpp_half_mirror(before);
                        if (PARTS >= 16) before += dpp_row_mirror(before);
                        if (c < n && part == 0) {
                            o_idx[before] = mine;
                            o_w[before] = u_w[c];
                        }
                    };
                    if (n <= 64u) file_by_index(std::integral_constant<uint32_t, 16>{});
                    else if (n <= 128u) file_by_index(std::integral_constant<uint32_t, 8>{});
                    else if (n <= 256u) file_by_index(std::integral_constant<uint32_t, 4>{});
                    else file_by_index(std::integral_constant<uint32_t, 2>{});
                    __syncthreads();
                }
                if (wave == 0) {
                    int64_t hit = -1;
                    uint64_t w_hit = 0;
                    if (seg >= 0 && seg < S_WAVES) {
                        uint64_t base = acc;
                        uint32_t rank0 = ties_before;
                        for (uint32_t q0 = 0; q0 < n; q0 += kWave) {  // wavefront-uniform
                            const bool live = q0 + uint32_t(lane) < n;
                            const uint32_t iw = live ? o_idx[q0 + lane] : 0u;
                            const uint64_t wv = live ? o_w[q0 + lane] : 0ull;
                            const bool tie = live && (iw >> 31) != 0;
                            const uint64_t tmask = __ballot(tie);
                            const uint32_t rank = rank0 + uint32_t(__popcll(tmask & ((uint64_t(1) << lane) - 1)));
                            const uint64_t weff = tie ? (rank < r_cut ? w_tie : 0ull) : wv;
                            const uint64_t inc = base + wave_incl_scan_u64(weff);
                            const uint64_t above = __ballot(live && inc > tau);
                            if (above != 0) {
                                const int f = __ffsll((long long)above) - 1;
                                hit = int64_t(uint32_t(__builtin_amdgcn_readlane(int(iw), f)) & 0x7fffffffu);
                                w_hit = (uint64_t(uint32_t(__builtin_amdgcn_readlane(int(uint32_t(weff >> 32)), f))) << 32) |
                                        uint32_t(__builtin_amdgcn_readlane(int(uint32_t(weff)), f));
                                break;
                            }
                            base = (uint64_t(uint32_t(__builtin_amdgcn_readlane(int(uint32_t(inc >> 32)), kWave - 1))) << 32) |
                                   uint32_t(__builtin_amdgcn_readlane(int(uint32_t(inc)), kWave - 1));
                            rank0 += uint32_t(__popcll(tmask));
                        }
                    } else if (seg == S_WAVES) {  // the ragged tail: fewer than eight entries, one per lane
                        const uint32_t rk = ties_before + wave_excl_scan<uint32_t>(tail_tie ? 1u : 0u);
                        const uint64_t wt = has_tail ? (tail_tie ? (rk < r_cut ? w_tie : 0ull)
                                                                 : (tail_key >= kcut16 ? table[tail_key >= first ? tail_key - kcut16 : span] : 0ull))
                                                     : 0ull;
                        const uint64_t before = acc + wave_excl_scan<uint64_t>(wt);
                        const uint64_t above = __ballot(before <= tau && tau < before + wt);
                        if (above != 0) {
                            const int f = __ffsll((long long)above) - 1;
                            hit = int64_t(nvec) * 8 + f;
                            w_hit = (uint64_t(uint32_t(__builtin_amdgcn_readlane(int(uint32_t(wt >> 32)), f))) << 32) |
                                    uint32_t(__builtin_amdgcn_readlane(int(uint32_t(wt)), f));
                        }
                    }
                    if (lane == 0) {
                        *out_slot = hit;
                        if (lp_slot != nullptr) *lp_slot = hit >= 0 ? log_ratio(w_hit, z) : __builtin_nanf("");
                    }
                    KA_STAMP(12);
                }
                return true;
            }
        }
    }
    // ---- 7. draw over the survivors in index order ------------------------------------------------------------
    auto mass = [&](uint32_t k) -> uint64_t {
        return all_survive ? table[idx16[k]] : table[k >= first ? k - kcut16 : span];
    };
    // 7a. per wavefront: mass of the full survivors and number of tie-group entries of its share of the row
    {
        uint64_t m = 0;
        uint32_t t = 0;
        for_wave_vectors<T, false>(vp, n_here, 1.0f, [&](bool valid, bool, const uint32_t (&kk)[4]) {
            if (valid) {
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    m += mass(key_at(kk, j));
                    t += is_tie(key_at(kk, j)) ? 1u : 0u;
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
    KA_STAMP(13);  // masses of every share
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
    // 7c. inside the segment (a wavefront's share of the row, in steps of 64 vectors): every wavefront sums one step,
    //     then the wavefront whose step holds tau finds the lane and the entry.  A share of more than S_WAVES steps
    //     (rows above 131,072 entries) takes further rounds of S_WAVES steps.
    if (seg >= 0 && seg < S_WAVES) {  // the same for the whole block
        const int sv0 = seg * vpw;
        const int n_seg = nvec - sv0 < vpw ? nvec - sv0 : vpw;
        const int n_steps = (n_seg + kWave - 1) / kWave;
        const int lane = tid & (kWave - 1);
        uint64_t cum = acc;
        uint32_t rank = ties_before;
        for (int st0 = 0; st0 < n_steps; st0 += S_WAVES) {  // block-uniform trip count and exit
            const int idx = (st0 + wave) * kWave + lane;
            const bool valid = idx < n_seg;
            uint32_t kk[4] = {0, 0, 0, 0}, k[8];
            uint64_t m = 0;
            uint32_t t = 0;
            if (st0 + wave < n_steps) {
                const uint4 q = valid ? (reinterpret_cast<const uint4 *>(rp) + sv0)[idx] : make_uint4(0, 0, 0, 0);
                vector_keys<T, false>(q, 1.0f, kk);
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) k[j] = key_at(kk, j);
            if (valid) {
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    m += mass(k[j]);
                    t += is_tie(k[j]) ? 1u : 0u;
                }
            }
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
                    uint32_t lt = 0;
#pragma unroll
                    for (int j = 0; j < 8; ++j) lt += (valid && is_tie(k[j])) ? 1u : 0u;
                    uint32_t rk = hrank + wave_excl_scan<uint32_t>(lt);
                    const uint32_t rk0 = rk;
                    uint64_t lm = 0;
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        if (valid) lm += is_tie(k[j]) ? ((rk++ < r_cut) ? w_tie : 0ull) : mass(k[j]);
                    const uint64_t before = hcum + wave_excl_scan<uint64_t>(lm);
                    if (before <= tau && tau < before + lm) {
                        uint64_t c2 = before;
                        uint32_t r2 = rk0;
                        bool done = false;
#pragma unroll
                        for (int j = 0; j < 8; ++j) {
                            const uint64_t wj = is_tie(k[j]) ? ((r2++ < r_cut) ? w_tie : 0ull) : mass(k[j]);
                            c2 += wj;
                            if (!done && c2 > tau) {
                                done = true;
                                ds.hit = (sv0 + idx) * 8 + j;
                                ds.pick_w = wj;
                            }
                        }
                    }
                }
                break;
            }
            __syncthreads();  // the per-step totals are overwritten by the next round
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
    KA_STAMP(14);  // entry located
    if (tid == 0) {
        *out_slot = ds.hit;
        if (lp_slot != nullptr) *lp_slot = ds.hit >= 0 ? log_ratio(ds.pick_w, z) : __builtin_nanf("");
    }
    return true;
}


}  // namespace
}  // namespace ka

#endif  // KA_SAMPLING_DENSE_H

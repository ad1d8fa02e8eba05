// Top-k route of the sampling kernel (1 <= top_k <= 1024): a short candidate list in LDS.
#ifndef KA_SAMPLING_TOPK_H
#define KA_SAMPLING_TOPK_H

#include "ka_sampling_common.h"

namespace ka {
namespace {

// ---------------------------------------------------------------------------
// Top-k route: everything after the first read of the row happens on a short candidate list in LDS.
//
//   1. maxima of disjoint shares of the row are taken while it streams by (each maximum is a different element);
//      the top_k-th largest of them, t, is a lower bound of the top_k-th largest element;
//   2. the bound is lowered to the smallest raw key that still scales to the same value as t (ties made
//      by the rounding of x / T must not be lost), and every element at or above it is collected:
//      a superset of the top-k survivors, ~top_k + a few entries on ordinary rows;
//   3. the candidates are scaled, ranked by (key desc, index asc), cut by top-k (ties kept) and top-p on
//      integer masses, and the draw is taken over the survivors in index order.
// Two routes do this (fast_topk below chooses; the caller can force the second): the short route for top_k <= 256
// (pooled maxima or a radix descent for the bound, candidate vectors re-read from L2, ranks by key and by index in one
// step, a scan-based tail on one wavefront) and the block-wide route (radix descent, row kept in registers where it
// fits, block-wide rank sort and scans).
// Returns false (having written nothing) when the candidates do not fit: the radix path then runs.
// All integer decisions are the same function of the row as in the radix path.
// ---------------------------------------------------------------------------

// ---------------------------------------------------------------------------
// Pieces of the short route (top_k <= SHORT_TOPK): after the read of the row, a handful of block-wide barriers and a tail on
// one wavefront instead of radix descents and block-wide scans.
// ---------------------------------------------------------------------------
constexpr int SHORT_TOPK = 256;      // largest top_k the short route serves
constexpr int SHORT_POOL_TOPK = 64;  // up to here the bound comes from pooled group maxima, above from a radix descent
constexpr int SHORT_GROUPS = 128;    // the lane maxima are pooled into this many group maxima (8 lanes each of 1024, 4 of 512)
constexpr int SHORT_POOL = S_THREADS / SHORT_GROUPS;  // lanes per group
constexpr int BLOCK_CAND = CAND_CAP < S_THREADS ? CAND_CAP : S_THREADS;  // candidates the block-wide tail ranks (one per thread)
static_assert(SHORT_POOL == 8 || SHORT_POOL == 4, "the pooling below is written for groups of 8 or 4 lanes");
constexpr int SHORT_VECS = 512;      // candidate vectors the short route takes (16 bytes each in LDS)
constexpr int SHORT_CAND = 512;      // candidates its tail takes (eight per lane of one wavefront)

// Minimum of one value per lane over the wavefront, in every lane (DPP row shifts and broadcasts, then lane 63).
template <int CTRL, int ROW_MASK> __device__ __forceinline__ uint32_t min_step_u32(uint32_t v) {
    const uint32_t o = uint32_t(__builtin_amdgcn_update_dpp(int(0xffffffffu), int(v), CTRL, ROW_MASK, 0xf, false));
    return o < v ? o : v;
}
__device__ __forceinline__ uint32_t wave_min_u32(uint32_t v) {
    v = min_step_u32<0x111, 0xf>(v);
    v = min_step_u32<0x112, 0xf>(v);
    v = min_step_u32<0x114, 0xf>(v);
    v = min_step_u32<0x118, 0xf>(v);
    v = min_step_u32<0x142, 0xa>(v);
    v = min_step_u32<0x143, 0xc>(v);
    return uint32_t(__builtin_amdgcn_readlane(int(v), kWave - 1));
}

// Where the short route keeps its lists in the candidate area of LDS once the candidates are ranked (step S5):
//   sh.c.raw[r], sh.c.sidx[r], sh.c.w[r]   scaled key, index and integer mass of the candidate of rank r, ranks by
//                                           (key descending, index ascending);
//   by_index_w(sh)[q], by_index_idx(sh)[q]  mass (0 until the tail files the kept ones) and index of the candidate
//                                           that is q-th in ascending index order.
__device__ __forceinline__ uint64_t *by_index_w(Shared &sh) { return sh.c.w + SHORT_CAND; }
__device__ __forceinline__ uint32_t *by_index_idx(Shared &sh) { return sh.c.sidx + SHORT_CAND; }
static_assert(2 * SHORT_CAND <= CAND_CAP && SHORT_VECS * 16 <= CAND_CAP * 8, "the short route's lists live in the candidate area");

// The tail of the short route on one wavefront, after the block has ranked the nc <= SHORT_CAND candidates both ways.
// Position p of the key order is handled by slot p / 64 of lane p % 64; na <= 64 * SLOTS positions hold the top-k
// survivors (ties kept).  Top-p cut on the prefix sums of the masses, then the kept masses are filed in index order
// and a second prefix sum finds the first index whose inclusive mass exceeds floor(u * Z): the same integer decisions
// as the block-wide tail, without a barrier and without a loop over pairs.
template <typename T, int SLOTS>
__device__ __forceinline__ void short_tail(Shared &sh, uint32_t nc, uint32_t na, const uint32_t *rank_by_index,
                                           bool use_p, float top_p, float u, int64_t *out_slot, float *lp_slot,
                                           const typename T::raw_t *rp, int vocab, float *policy_slot, const PolicyLse &lse) {
    const int lane = threadIdx.x & (kWave - 1);
    uint64_t w[SLOTS], before[SLOTS];
    uint64_t carry = 0;
#pragma unroll
    for (int s = 0; s < SLOTS; ++s) {
        const uint32_t p = uint32_t(s * kWave + lane);
        w[s] = p < na ? sh.c.w[p] : 0ull;
        const uint64_t inc = wave_incl_scan_u64(w[s]);
        before[s] = carry + inc - w[s];
        carry += (uint64_t(uint32_t(__builtin_amdgcn_readlane(int(uint32_t(inc >> 32)), kWave - 1))) << 32) |
                 uint32_t(__builtin_amdgcn_readlane(int(uint32_t(inc)), kWave - 1));
    }
    const uint64_t z_topk = carry;
    KA_STAMP(6);   // prefix of the masses
    // top-p: `before` is non-decreasing along the key order, so the kept entries are a prefix; its mass is the
    // inclusive sum at its last position.  Kept masses go to their place in index order.
    uint64_t z_kept = 0;
    {
        const uint64_t theta = use_p ? floor_scale(top_p, z_topk) : ~0ull;
        uint64_t *const wq = by_index_w(sh);
#pragma unroll
        for (int s = 0; s < SLOTS; ++s) {
            const uint32_t p = uint32_t(s * kWave + lane);
            const bool kept = p < na && before[s] <= theta;
            const int n_here = __popcll(__ballot(kept));
            if (n_here > 0) {
                const uint64_t upto = before[s] + w[s];
                z_kept = (uint64_t(uint32_t(__builtin_amdgcn_readlane(int(uint32_t(upto >> 32)), n_here - 1))) << 32) |
                         uint32_t(__builtin_amdgcn_readlane(int(uint32_t(upto)), n_here - 1));
            }
            if (kept) wq[rank_by_index[p]] = w[s];
        }
    }
    KA_STAMP(7);   // top-p cut
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // draw: inclusive mass in index order; the first position above floor(u * Z) wins
    const uint64_t tau = floor_scale(u, z_kept);
    uint32_t hit = 0xffffffffu;
    uint64_t w_hit = 0;
    {
        const uint64_t *const wq = by_index_w(sh);
        const uint32_t *const iq = by_index_idx(sh);
        uint64_t base = 0;
        for (uint32_t q0 = 0; q0 < nc; q0 += kWave) {  // wavefront-uniform: one to four rounds
            const uint32_t q = q0 + uint32_t(lane);
            const uint64_t wv = q < nc ? wq[q] : 0ull;
            const uint64_t inc = base + wave_incl_scan_u64(wv);
            const uint64_t above = __ballot(inc > tau);
            if (above != 0) {
                const int first = __ffsll((long long)above) - 1;
                hit = iq[q0 + uint32_t(first)];
                w_hit = (uint64_t(uint32_t(__builtin_amdgcn_readlane(int(uint32_t(wv >> 32)), first))) << 32) |
                        uint32_t(__builtin_amdgcn_readlane(int(uint32_t(wv)), first));
                break;
            }
            base = (uint64_t(uint32_t(__builtin_amdgcn_readlane(int(uint32_t(inc >> 32)), kWave - 1))) << 32) |
                   uint32_t(__builtin_amdgcn_readlane(int(uint32_t(inc)), kWave - 1));
        }
    }
    KA_STAMP(8);   // draw
    if (lane == 0) {
        *out_slot = hit == 0xffffffffu ? int64_t(-1) : int64_t(hit);
        if (lp_slot != nullptr) *lp_slot = hit == 0xffffffffu ? __builtin_nanf("") : log_ratio(w_hit, z_kept);
        if (policy_slot != nullptr) *policy_slot = lse.template finish<T>(rp, hit == 0xffffffffu ? int64_t(-1) : int64_t(hit), vocab);
    }
}

// Returns 0 (nothing written: the radix path runs), 1 (id and filtered log-probability written) or 2 (the policy
// log-probability as well: the short route takes the row's log-sum-exp along while the row streams by).
template <typename T>
__device__ __forceinline__ int fast_topk(Shared &sh, const typename T::raw_t *rp, int vocab, bool vec, float temp,
                                         bool has_t, int top_k, bool use_p, float top_p, float u,
                                         int64_t *out_slot, float *lp_slot, bool block_wide_only, float *policy_slot,
                                         PolicyLse &lse) {
    const int tid = threadIdx.x;
    // top_k <= 64 takes the short route unless the caller asks for the block-wide one (the two give the same ids)
    // (the build with 512 threads has no block-wide route: what its short route cannot take goes to the radix path)
    if (S_THREADS != 1024 && (top_k > SHORT_TOPK || block_wide_only)) return 0;
    const bool short_route = top_k <= SHORT_TOPK && !block_wide_only;
    // 1. lane maxima of the raw values (float max: one convert and half a v_max3 per element; which of
    //    -0 / +0 it returns does not matter, any lower bound of the top_k-th element will do)
    //    On the block-wide route a row that fits (16-byte aligned, at most 16 vectors per lane: 131,072 bf16 entries)
    //    is kept in registers, so that the collection pass below reads nothing from memory.  The short route keeps
    //    32 maxima per lane instead and re-reads the few vectors that hold a candidate from L2: with 64 of a lane's
    //    128 registers holding the row, its selection code spills, and the spills cost more than the re-reads.
    constexpr int EPV = T::kPerVec;
    constexpr int RES_VECS = 16;
    const int nvec = vocab / EPV;
    const bool resident = !short_route && vec && T::kDtype == KA_DTYPE_BF16 && nvec <= RES_VECS * S_THREADS;
    // A longer or wider row does not fit in registers, but 32 maxima per lane do: slot r keeps the maximum of the
    // lane's vectors tid + (g * 32 + r) * 1024, g = 0 .. trk_rounds - 1, and the collection pass re-reads only the
    // slots that hold a candidate.  One vector per slot covers an fp32 row of 131,072 entries and a 16-bit row of
    // 262,144; longer fp32 rows take up to four vectors per slot (for the 16-bit dtypes the count stays a
    // compile-time 1, which keeps their kernels as they are).  (A resident row keeps no per-vector maxima: with the
    // row in 64 registers of the 128 a lane has, sixteen more spill and slow the read down.)
    constexpr int TRK_VECS = 32;
    constexpr int TRK_BATCH = 8;  // loads in flight per lane (with 16, the 128 registers of a lane spill)
    const int trk_need = (nvec + TRK_VECS * S_THREADS - 1) / (TRK_VECS * S_THREADS);
    const int trk_rounds = T::kBytes == 4 ? trk_need : 1;
    const bool tracked = vec && !resident && trk_need <= (T::kBytes == 4 ? 4 : 1);
    // the short route folds the row's log-sum-exp while it reads a row it tracks (the order of row_lse_to_block, so the
    // value does not depend on the route); other rows get the fold's own pass at the end of the kernel
    const bool take_lse = short_route && policy_slot != nullptr && tracked;
    ThreadLse acc_lse;
    uint4 held[RES_VECS];
    // The slot maxima of a 16-bit row are kept in the row's own 16 bits, two per register (they are elements of the
    // row, so nothing is lost): 32 floats next to the loads in flight would spill.
    constexpr bool PACKED = T::kBytes == 2;
    uint32_t vstore[PACKED ? TRK_VECS / 2 : TRK_VECS];
    auto narrow16 = [](float v) -> uint32_t {
        if (T::kDtype == KA_DTYPE_F16) {
            union { _Float16 h; uint16_t u; } c;
            c.h = _Float16(v);
            return c.u;
        }
        return __float_as_uint(v) >> 16;
    };
    auto set_slot_max = [&](int slot, float vm, bool first_round) {  // slot is a compile-time value at every call
        if (PACKED) {
            if ((slot & 1) == 0) vstore[slot / 2] = narrow16(vm);
            else vstore[slot / 2] |= narrow16(vm) << 16;
        } else {
            vstore[slot] = __float_as_uint(first_round ? vm : fmaxf(__uint_as_float(vstore[slot]), vm));
        }
    };
    auto slot_max = [&](int slot) -> float {
        if (PACKED) return T::widen(typename T::raw_t((slot & 1) == 0 ? (vstore[slot / 2] & 0xffffu) : (vstore[slot / 2] >> 16)));
        return __uint_as_float(vstore[slot]);
    };
    float lmaxf = -__builtin_inff();
    auto vector_max = [](const uint4 &q) { return ka::vector_max<T>(q); };
    if (tracked) {
        const uint4 *vp = reinterpret_cast<const uint4 *>(rp);
#pragma unroll 1
        for (int round = 0; round < trk_rounds; ++round) {
            const int base = tid + round * TRK_VECS * S_THREADS;
#pragma unroll
            for (int g = 0; g < TRK_VECS / TRK_BATCH; ++g) {
                if ((round * TRK_VECS + g * TRK_BATCH) * S_THREADS >= nvec) {  // block-uniform: nothing of the row is left
                    if (round == 0) {
#pragma unroll
                        for (int s = 0; s < TRK_BATCH; ++s) set_slot_max(g * TRK_BATCH + s, -__builtin_inff(), true);
                    }
                    continue;
                }
                uint4 q[TRK_BATCH];
#pragma unroll
                for (int s = 0; s < TRK_BATCH; ++s) {
                    const int v = base + (g * TRK_BATCH + s) * S_THREADS;
                    q[s] = v < nvec ? vp[v] : make_uint4(0, 0, 0, 0);
                }
#pragma unroll
                for (int s = 0; s < TRK_BATCH; ++s) {
                    float vm = -__builtin_inff();
                    if (base + (g * TRK_BATCH + s) * S_THREADS < nvec) {
                        vm = vector_max(q[s]);
                        if (take_lse) {
                            float x[EPV];
                            T::unpack(q[s], x);
                            acc_lse.lane[(g * TRK_BATCH + s) % LSE_PER_THREAD].add_vector(x, vm);
                        }
                    }
                    set_slot_max(g * TRK_BATCH + s, vm, round == 0);
                    lmaxf = fmaxf(lmaxf, vm);
                }
            }
        }
        const int i = nvec * EPV + tid;  // ragged tail of the row
        if (i < vocab) {
            lmaxf = fmaxf(lmaxf, T::widen(rp[i]));
            if (take_lse) acc_lse.lane[0].add(T::widen(rp[i]));
        }
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
        for_each_raw<T, 8>(rp, vocab, vec, [&](int, typename T::raw_t raw) {
            lmaxf = fmaxf(lmaxf, T::widen(raw));
        });
    }
    if (take_lse) acc_lse.to_block(lse);  // a barrier follows on every way on (pooling of the maxima, radix descent)
    KA_STAMP(1);   // row read, lane maxima known
    // 2. (both routes) the bound is widened over the raw values that scale to the same value; false: a huge
    //    temperature folds too many values together
    auto widen_bound = [&](uint32_t &bound) {
        if (!has_t) return true;
        // Lane l scales the value l steps below the bound; scaling is monotone, so the lanes whose scaled value still
        // equals the bound's form a prefix, and its length says how far the bound moves.  (One division per lane instead of
        // a loop of dependent ones; every wavefront does the same work.)  All 64 lanes equal: a huge temperature.
        const int l = tid & (kWave - 1);
        const uint32_t mine = bound - uint32_t(l) * key_step<T>();
        const bool valid = bound >= uint32_t(l) * key_step<T>();
        const uint32_t key = elem_key<T>(raw_of_key<T>(valid ? mine : bound), temp, true);
        const uint32_t ty = uint32_t(__builtin_amdgcn_readfirstlane(int(key)));
        const uint64_t same = __ballot(valid && key >= ty);
        if (~same == 0) return false;
        const int n = __ffsll((long long)~same) - 1;  // length of the prefix; >= 1: lane 0
        bound -= uint32_t(n - 1) * key_step<T>();
        return true;
    };
    // the top_k-th largest of the 1024 lane maxima, by the same MSB-first descent over count histograms as the radix path
    auto radix_bound = [&]() -> uint32_t {
        const uint32_t lmax = masked_key<T>(lmaxf);
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
        return prefix << level_shift<T>(Round<T>::kLevels - 1);
    };
    bool have_candidates = false;  // the short route has filled the candidate list but leaves the tail to the block
    if (short_route) {
        uint32_t bound;
        if (top_k <= SHORT_POOL_TOPK) {
        // S1. The lane maxima are pooled into 128 group maxima (eight neighbouring lanes each); the top_k-th largest
        //     group maximum is a lower bound of the top_k-th largest element (each group maximum is a different
        //     element), and with top_k well below 128 nearly as tight as the top_k-th largest lane maximum.
        float gmax = lmaxf;
        gmax = fmaxf(gmax, __uint_as_float(dpp_xor1(__float_as_uint(gmax))));
        gmax = fmaxf(gmax, __uint_as_float(dpp_xor2(__float_as_uint(gmax))));
        if (SHORT_POOL == 8) gmax = fmaxf(gmax, __uint_as_float(dpp_half_mirror(__float_as_uint(gmax))));
        if ((tid & (SHORT_POOL - 1)) == 0) sh.c.skey[tid / SHORT_POOL] = __float_as_uint(gmax);
        if (tid == 0) { sh.n_cand = 0; sh.n_vec = 0; sh.hit = -1; sh.cand_kmax = 0; }
        __syncthreads();
        // S2. Eight threads rank one group maximum among the 128 (descending, ties by position): sixteen compares
        //     each, summed inside the group of eight lanes.  Exactly one maximum has rank top_k - 1.
        {
            constexpr int SHARE = SHORT_GROUPS / SHORT_POOL;  // group maxima one thread compares against
            const int v = tid / SHORT_POOL, part = tid & (SHORT_POOL - 1);
            const float x = __uint_as_float(sh.c.skey[v]);
            const uint4 *others = reinterpret_cast<const uint4 *>(sh.c.skey + part * SHARE);
            uint32_t cnt = 0;
#pragma unroll
            for (int q = 0; q < SHARE / 4; ++q) {
                const uint4 o = others[q];
                const uint32_t ow[4] = {o.x, o.y, o.z, o.w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float of = __uint_as_float(ow[e]);
                    const int j = part * SHARE + q * 4 + e;
                    cnt += (of > x || (of == x && j < v)) ? 1u : 0u;
                }
            }
            cnt += dpp_xor1(cnt);
            cnt += dpp_xor2(cnt);
            if (SHORT_POOL == 8) cnt += dpp_half_mirror(cnt);
            if (part == 0 && cnt == uint32_t(top_k - 1)) sh.max_key = __float_as_uint(x);
        }
        __syncthreads();
        bound = masked_key<T>(__uint_as_float(sh.max_key));
        } else {
            // 64 < top_k <= 256: the exact top_k-th largest lane maximum (128 pooled maxima would be too few)
            bound = radix_bound();
            if (tid == 0) { sh.n_cand = 0; sh.n_vec = 0; sh.hit = -1; sh.cand_kmax = 0; }
            __syncthreads();
        }
        KA_STAMP(2);   // bound known
        if (!widen_bound(bound)) return 0;
        KA_STAMP(3);   // bound widened
        const float boundf = value_of<T>(bound);  // a float compare admits -0 next to +0: still a superset
        // Fewer than top_k groups hold a number above -inf: the survivors may include -inf entries (and NaNs, which
        // count as -inf but fail every float compare).  Leave such rows to the radix path.
        if (boundf == -__builtin_inff()) return 0;
        // S3. Vectors that hold a candidate go to a list in LDS whole (one atomic per vector, nothing per element
        //     in the wavefronts that hold the row); single elements (ragged tail, unaligned rows) go straight to the
        //     candidate list with their scaled key.
        uint4 *const cvec = reinterpret_cast<uint4 *>(sh.c.w);  // [SHORT_VECS] vectors ...
        uint32_t *const cvidx = sh.c.sidx;                      // ... and their vector numbers
        auto add_vector = [&](int v, const uint4 &q) {
            const uint32_t slot = atomicAdd(&sh.n_vec, 1u);
            if (slot < uint32_t(SHORT_VECS)) {
                cvec[slot] = q;
                cvidx[slot] = uint32_t(v);
            }
        };
        auto add_element = [&](int i, typename T::raw_t raw) {
            if (T::widen(raw) >= boundf) {
                const uint32_t slot = atomicAdd(&sh.n_cand, 1u);
                if (slot < CAND_CAP) {
                    const uint32_t key = elem_key<T>(raw, temp, has_t);
                    sh.c.raw[slot] = uint32_t(raw);
                    sh.c.idx[slot] = uint32_t(i);
                    sh.c.skey[slot] = key;
                    atomicMax(&sh.cand_kmax, key);  // the row maximum is a candidate: the largest candidate key is its key
                }
            }
        };
        if (tracked) {
            // Slots whose maximum reaches the bound (about top_k of the 32,768 slots of a row do).  Every lane then
            // works through its own hits, one per turn, so that the loads of a wavefront go out together: a lane
            // rarely has more than one, and a wavefront takes as many turns as its busiest lane has hits.
            const uint4 *vp = reinterpret_cast<const uint4 *>(rp);
            uint32_t hits = 0;
#pragma unroll
            for (int r = 0; r < TRK_VECS; ++r) hits |= slot_max(r) >= boundf ? 1u << r : 0u;
            while (__any(hits != 0)) {
                if (hits != 0) {
                    const int r = __ffs(hits) - 1;
                    hits &= hits - 1;
                    for (int round = 0; round < trk_rounds; ++round) {
                        const int v = tid + (round * TRK_VECS + r) * S_THREADS;
                        if (v < nvec) {
                            const uint4 q = vp[v];
                            if (trk_rounds == 1 || vector_max(q) >= boundf) add_vector(v, q);
                        }
                    }
                }
            }
            const int i = nvec * EPV + tid;
            if (i < vocab) add_element(i, rp[i]);
        } else {
            for_each_raw<T, 8>(rp, vocab, vec, add_element);
        }
        __syncthreads();
        KA_STAMP(4);   // candidate vectors collected
        const uint32_t nv = sh.n_vec;
        if (nv <= uint32_t(SHORT_VECS)) {
            // S4. One thread per element of the listed vectors: those at or above the bound join the candidate list.
            for (int i = tid; i < int(nv) * EPV; i += S_THREADS) {
                const int vslot = i / EPV, e = i % EPV;
                const typename T::raw_t raw = reinterpret_cast<const typename T::raw_t *>(cvec + vslot)[e];
                add_element(int(cvidx[vslot]) * EPV + e, raw);
            }
            __syncthreads();
            KA_STAMP(10);  // candidates expanded
            const uint32_t nc = sh.n_cand;
            if (nc > CAND_CAP) return 0;
            if (nc <= uint32_t(SHORT_CAND)) {
                // S5. Four threads rank one candidate twice, by (scaled key descending, index ascending) and by index
                //     alone, and file it under both ranks together with its integer mass (see by_index_w above; none
                //     of the arrays written here is read in this step).
                uint32_t *const rank_by_index = sh.c.raw + SHORT_CAND;  // [key rank] -> position in index order
                // PARTS threads share a candidate (16 for up to 64 candidates, 8 up to 128, 4 up to 256, 2 up to 512: all 1024
                // threads take part), each over every PARTS-th group of four entries; the counts are summed inside the
                // PARTS neighbouring lanes by DPP.
                auto rank_candidates = [&](auto parts_c) {
                    constexpr uint32_t PARTS = decltype(parts_c)::value;
                    const uint32_t c = uint32_t(tid) / PARTS, part = uint32_t(tid) % PARTS;
                    uint32_t ki = 0, ii = 0, cnt = 0, cnt_i = 0;
                    if (c < nc) {
                        ki = sh.c.skey[c];
                        ii = sh.c.idx[c];
                        // 16-byte reads; entries past nc are stale but inside the list and masked out below
                        const uint4 *k4 = reinterpret_cast<const uint4 *>(sh.c.skey);
                        const uint4 *i4 = reinterpret_cast<const uint4 *>(sh.c.idx);
                        for (uint32_t m = part; m * 4 < nc; m += PARTS) {
                            const uint4 kq = k4[m], iq = i4[m];
                            const uint32_t kk[4] = {kq.x, kq.y, kq.z, kq.w}, ik[4] = {iq.x, iq.y, iq.z, iq.w};
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                const bool live = m * 4 + e < nc;
                                cnt += (live && (kk[e] > ki || (kk[e] == ki && ik[e] < ii))) ? 1u : 0u;
                                cnt_i += (live && ik[e] < ii) ? 1u : 0u;
                            }
                        }
                    }
                    uint32_t both = cnt | (cnt_i << 16);  // both counts stay below 2^16: one register through the DPP sums
                    if (PARTS >= 2) both += dpp_xor1(both);
                    if (PARTS >= 4) both += dpp_xor2(both);
                    if (PARTS >= 8) both += dpp_half_mirror(both);
                    if (PARTS >= 16) both += dpp_row_mirror(both);
                    cnt = both & 0xffffu;
                    cnt_i = both >> 16;
                    if (c < nc && part == 0) {
                        const uint32_t kmax = sh.cand_kmax;
                        sh.c.raw[cnt] = ki;
                        sh.c.sidx[cnt] = ii;
                        sh.c.w[cnt] = weight_fix(ki == kmax ? 0.0f : value_of<T>(ki) - value_of<T>(kmax));
                        rank_by_index[cnt] = cnt_i;
                        by_index_w(sh)[cnt_i] = 0;
                        by_index_idx(sh)[cnt_i] = ii;
                    }
                };
                if (nc <= 64u) rank_candidates(std::integral_constant<uint32_t, S_THREADS / 64>{});
                else if (nc <= 128u) rank_candidates(std::integral_constant<uint32_t, S_THREADS / 128>{});
                else if (nc <= 256u) rank_candidates(std::integral_constant<uint32_t, S_THREADS / 256>{});
                else rank_candidates(std::integral_constant<uint32_t, S_THREADS / 512>{});
                __syncthreads();
                KA_STAMP(5);   // candidates sorted
                if (tid < kWave) {  // one wavefront finishes the row; the others are done
                    // entries behind the top-k survivors play no part: the tail is sized by their number
                    const uint32_t kstar = sh.c.raw[top_k - 1];
                    uint32_t na = 0;
#pragma unroll
                    for (int s = 0; s < SHORT_CAND / kWave; ++s) {
                        const uint32_t pp = uint32_t(s * kWave + tid);
                        na += uint32_t(__popcll(__ballot(pp < nc && sh.c.raw[pp] >= kstar)));
                    }
                    if (na <= uint32_t(kWave)) short_tail<T, 1>(sh, nc, na, rank_by_index, use_p, top_p, u, out_slot, lp_slot, rp, vocab, take_lse ? policy_slot : nullptr, lse);
                    else if (na <= uint32_t(2 * kWave)) short_tail<T, 2>(sh, nc, na, rank_by_index, use_p, top_p, u, out_slot, lp_slot, rp, vocab, take_lse ? policy_slot : nullptr, lse);
                    else if (na <= uint32_t(4 * kWave)) short_tail<T, 4>(sh, nc, na, rank_by_index, use_p, top_p, u, out_slot, lp_slot, rp, vocab, take_lse ? policy_slot : nullptr, lse);
                    else short_tail<T, 8>(sh, nc, na, rank_by_index, use_p, top_p, u, out_slot, lp_slot, rp, vocab, take_lse ? policy_slot : nullptr, lse);
                    KA_STAMP(9);
                }
                return take_lse ? 2 : 1;
            }
            if (S_THREADS != 1024) return 0;
            have_candidates = true;  // more than 512 candidates (a large tie group): the block-wide tail ranks them
        }
        if (S_THREADS != 1024) return 0;
        __syncthreads();  // too many candidate vectors: the block-wide route starts over with its exact bound
    }
    if (!have_candidates) {
    uint32_t bound = radix_bound();
    if (tid == 0) { sh.n_cand = 0; sh.hit = -1; }
    __syncthreads();
    KA_STAMP(2);   // bound known
    if (!widen_bound(bound)) return 0;
    KA_STAMP(3);   // bound widened
    const float boundf = value_of<T>(bound);  // a float compare admits -0 next to +0: still a superset
    // Fewer than top_k lanes hold a number above -inf: the survivors then include -inf entries (and NaNs,
    // which count as -inf but fail every float compare).  Leave such rows to the radix path.
    if (boundf == -__builtin_inff()) return 0;
    auto collect = [&](int i, typename T::raw_t raw) {
        if (T::widen(raw) >= boundf) {
            const uint32_t slot = atomicAdd(&sh.n_cand, 1u);
            if (slot < CAND_CAP) {
                sh.c.raw[slot] = uint32_t(raw);
                sh.c.idx[slot] = uint32_t(i);
            }
        }
    };
    // (after a fall-back from the short route the row is read again rather than kept in registers all the way here)
    if (resident && !short_route) {
#pragma unroll
        for (int r = 0; r < RES_VECS; ++r) {
            if (tid + r * S_THREADS < nvec && vector_max(held[r]) >= boundf) {  // rare: about top_k vectors of the row hold a candidate
                const typename T::raw_t *e = reinterpret_cast<const typename T::raw_t *>(&held[r]);
#pragma unroll
                for (int j = 0; j < EPV; ++j) collect((tid + r * S_THREADS) * EPV + j, e[j]);
            }
        }
        const int i = nvec * EPV + tid;
        if (i < vocab) collect(i, rp[i]);
    } else if (tracked && !short_route) {
        const uint4 *vp = reinterpret_cast<const uint4 *>(rp);
#pragma unroll
        for (int r = 0; r < TRK_VECS; ++r) {
            if (slot_max(r) >= boundf) {  // rare: about top_k slots of the whole row hold a candidate
                for (int round = 0; round < trk_rounds; ++round) {
                    const int v = tid + (round * TRK_VECS + r) * S_THREADS;
                    if (v < nvec) {
                        const uint4 q = vp[v];
                        const typename T::raw_t *e = reinterpret_cast<const typename T::raw_t *>(&q);
#pragma unroll
                        for (int j = 0; j < EPV; ++j) collect(v * EPV + j, e[j]);
                    }
                }
            }
        }
        const int i = nvec * EPV + tid;
        if (i < vocab) collect(i, rp[i]);
    } else {
        for_each_raw<T, 8>(rp, vocab, vec, collect);
    }
    __syncthreads();
    KA_STAMP(4);   // candidates collected
    }
    const uint32_t nc = sh.n_cand;
    if (nc > BLOCK_CAND) return 0;
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
    KA_STAMP(5);
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
    KA_STAMP(7);
    // 3d. draw: inclusive mass over the survivors in index order; the first index above floor(u * Z) wins
    const uint64_t tau = floor_scale(u, z_kept);
    if (tid < int(nb)) {
        const uint32_t mine = sh.c.sidx[tid];
        uint64_t cum = 0;
        for (uint32_t j = 0; j < nb; ++j) cum += sh.c.sidx[j] <= mine ? sh.c.w[j] : 0ull;
        if (cum > tau) atomicMin(reinterpret_cast<unsigned long long *>(&sh.hit), (unsigned long long)mine);
    }
    __syncthreads();
    KA_STAMP(9);
    if (tid == 0) *out_slot = sh.hit;
    if (lp_slot != nullptr && tid < int(nb) && int64_t(sh.c.sidx[tid]) == sh.hit) *lp_slot = log_ratio(sh.c.w[tid], z_kept);
    return 1;
}


}  // namespace
}  // namespace ka

#endif  // KA_SAMPLING_TOPK_H

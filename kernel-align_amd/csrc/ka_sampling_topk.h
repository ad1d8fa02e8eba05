// Top-k fast path of the sampling kernel (1 <= top_k <= 1024): a short candidate list in LDS.
#ifndef KA_SAMPLING_TOPK_H
#define KA_SAMPLING_TOPK_H

#include "ka_sampling_common.h"

namespace ka {
namespace {

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
    // A longer or wider row does not fit in registers, but 32 maxima per lane do: slot r keeps the maximum of the
    // lane's vectors tid + (g * 32 + r) * 1024, g = 0 .. trk_rounds - 1, and the collection pass re-reads only the
    // slots that hold a candidate.  One vector per slot covers an fp32 row of 131,072 entries and a 16-bit row of
    // 262,144; longer fp32 rows take up to four vectors per slot (for the 16-bit dtypes the count stays a
    // compile-time 1, which keeps their kernels as they are).
    constexpr int TRK_VECS = 32;
    const int trk_need = (nvec + TRK_VECS * S_THREADS - 1) / (TRK_VECS * S_THREADS);
    const int trk_rounds = T::kBytes == 4 ? trk_need : 1;
    const bool tracked = vec && !resident && trk_need <= (T::kBytes == 4 ? 4 : 1);
    uint4 held[RES_VECS];
    float vmaxs[TRK_VECS];
    float lmaxf = -__builtin_inff();
    if (tracked) {
        const uint4 *vp = reinterpret_cast<const uint4 *>(rp);
#pragma unroll 1
        for (int round = 0; round < trk_rounds; ++round) {
            const int base = tid + round * TRK_VECS * S_THREADS;
#pragma unroll
            for (int g = 0; g < TRK_VECS / 8; ++g) {
                uint4 q[8];
#pragma unroll
                for (int s = 0; s < 8; ++s) {
                    const int v = base + (g * 8 + s) * S_THREADS;
                    q[s] = v < nvec ? vp[v] : make_uint4(0, 0, 0, 0);
                }
#pragma unroll
                for (int s = 0; s < 8; ++s) {
                    float vm = -__builtin_inff();
                    if (base + (g * 8 + s) * S_THREADS < nvec) {
                        const typename T::raw_t *e = reinterpret_cast<const typename T::raw_t *>(&q[s]);
#pragma unroll
                        for (int j = 0; j < EPV; ++j) vm = fmaxf(vm, T::widen(e[j]));
                    }
                    vmaxs[g * 8 + s] = round == 0 ? vm : fmaxf(vmaxs[g * 8 + s], vm);
                    lmaxf = fmaxf(lmaxf, vm);
                }
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
            if (vmaxs[r] >= boundf) {  // rare: about top_k slots of the whole row hold a candidate
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


}  // namespace
}  // namespace ka

#endif  // KA_SAMPLING_TOPK_H

// Fused lm_head -> logprob: out[n] = h_n . W[id_n] - logsumexp_v(h_n . W[v]),
// without materialising the [n_rows, vocab] logits.
//
// Tiling (gfx950, wave64, v_mfma_f32_32x32x16_bf16):
//   * one workgroup of 4 wavefronts per CU walks work items; an item is 256
//     tokens x a range of 256-row vocabulary tiles; per tile it runs a K loop over the hidden dimension in
//     slabs of 64 (one cache line per row); the W slab [256 x 64] and the hidden
//     slab [256 x 64] go from global memory straight into XOR-swizzled LDS
//     (global_load_lds_dwordx4, no register staging), two stages of 64 KB, one
//     barrier per slab, three quarters into it; fragment reads run one k-step
//     ahead of the MFMAs;
//   * the MFMA "A" operand is W (rows of the result = vocabulary entries) and
//     "B" is hidden (columns = tokens), so every lane's 64 accumulators of one
//     32-column block belong to ONE token: the online max / sum-of-exp update
//     after each vocabulary tile is register-local, with no cross-lane traffic;
//   * each wavefront computes 128 vocab x 128 tokens = 4 x 4 MFMA blocks
//     (256 fp32 accumulators per lane);
//   * the vocabulary is cut into fixed splits of at most LM_TILES_PER_SPLIT tiles and every split into LM_SUBS
//     units of at most two tiles (a function of the vocabulary only).  A row's result is defined as: per unit an
//     online (max, sum, target logit), the units of a split folded in order, the splits folded in order - so it
//     does not depend on the number of rows, nor on who folds: with many rows an item is a (token block, split)
//     pair and the kernel folds the units itself; with few rows (fewer items than CUs) an item is a
//     (token block, unit) pair, so that one token block occupies every CU, and the second kernel folds the
//     units with the same operations.  Same bits either way.
// Logits stay in fp32 (the accumulators are not rounded to bf16).
#include <mutex>

#include "ka_common.h"

namespace ka {
namespace {

constexpr int LM_BM = 256;      // vocabulary rows per tile
constexpr int LM_BN = 256;      // tokens per workgroup
constexpr int LM_BK = 64;       // hidden slab: one 128-byte line per row
constexpr int LM_STAGES = 2;    // LDS: the slab in use and the slab in flight
constexpr int LM_STAGE_ELEMS = (LM_BM + LM_BN) * LM_BK;  // bf16 elements per LDS stage (64 KB)
constexpr int LM_XCH_BYTES = 2 * 4 * 32 * 4 * 4;  // exchange area of the end-of-unit fold: [wave_n][tn][32 lanes][4 floats]
constexpr int LM_SPLIT_ACC_BYTES = LM_XCH_BYTES;  // running partial of the item's split, same shape (touched by its own lane only)
constexpr int LM_LDS_BYTES = LM_STAGES * LM_STAGE_ELEMS * 2 + LM_XCH_BYTES + LM_SPLIT_ACC_BYTES;
constexpr int LM_THREADS = 256;
// Vocabulary tiles per split (at most).  Short splits let a single token block occupy many CUs: at
// V = 128,256 (501 tiles, 64 splits of 7 or 8) 64 rows take 0.74 ms, against 5.3 ms with 63 tiles per split.
constexpr int LM_TILES_PER_SPLIT = 8;
// Units per split.  With 8-tile splits a unit is two tiles: at V = 128,256 a single token block then makes 256 items,
// one per CU, of 1 - 2 tiles each (64 rows: 0.73 ms with whole splits as items).
constexpr int LM_SUBS = 4;
// Group (of 32 per slab) at which the next slab is waited for.  It lies in the last k-step: the first fragments of
// the next slab are loaded into the buffer that the k-steps 0 and 2 read, right behind the barrier.  (28 measures 2 %
// slower.)
constexpr int LM_BAR = 24;
// When the sixteen copies of a slab are requested.  A slab's window opens behind the barrier that frees its stage
// (group LM_BAR of the slab two before it) and closes at the next barrier, 32 groups later; copy c is requested at
// position c of the window, i.e. in group (LM_BAR + c) % 32: one copy per group over the first half of the window
// (spreading them over the whole window, or two per group, measured slower).
struct CopyTable {  // [group]: the copy requested in that group, -1 = none (a table: the group loop must stay cheap to unroll)
    signed char at[32];
    constexpr CopyTable() : at{} {
        for (int g = 0; g < 32; ++g) {
            const int pos = g >= LM_BAR ? g - LM_BAR : g + 32 - LM_BAR;
            at[g] = (signed char)(pos < 16 ? pos : -1);
        }
    }
};
constexpr CopyTable kCopyTable{};
constexpr int LM_FIRST = 32 - LM_BAR;  // copies of a slab requested before the slab boundary (groups LM_BAR .. 31)
// Group in which the copy cursor moves on to the next slab: between the last copy of a window and the first of the
// next one.
constexpr int LM_ADV = 12;
static_assert(LM_BAR >= 24 && LM_BAR <= 28, "the barrier group must lie in the last k-step and leave four groups for the reads");
static_assert(LM_ADV <= LM_BAR && LM_ADV + 32 - LM_BAR > 15, "the cursor moves between two windows");
constexpr float kLog2e = 1.44269504088896340736f;
constexpr double kLn2 = 0.693147180559945309417232;
constexpr float kFloor = -1.0e30f;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// The split plan is a function of the vocabulary only, so no row's result depends on the number of rows: a
// multiple of 8 splits (the width of a super-tile) of nearly equal size, none above LM_TILES_PER_SPLIT tiles.
__host__ __device__ inline int lm_n_splits(int n_vtiles) {
    return n_vtiles <= 8 ? n_vtiles : 8 * ((n_vtiles + 8 * LM_TILES_PER_SPLIT - 1) / (8 * LM_TILES_PER_SPLIT));
}
// The plan in the form the kernels use (no division on the device): every split holds `base` tiles, the first `rem`
// splits one more.
struct SplitPlan {
    int n_vtiles, n_splits, base, rem;
    __host__ __device__ SplitPlan(int n_vtiles_, int n_splits_)
        : n_vtiles(n_vtiles_), n_splits(n_splits_), base(n_vtiles_ / n_splits_), rem(n_vtiles_ % n_splits_) {}
    // First vocabulary tile of split sp (sp == n_splits: the end).
    __host__ __device__ int split_begin(int sp) const { return sp * base + (sp < rem ? sp : rem); }
    // First vocabulary tile of unit u = split * LM_SUBS + j (u == n_splits * LM_SUBS: the end).  Units of a split
    // shorter than LM_SUBS tiles may be empty.
    __host__ __device__ int unit_begin(int u) const {
        const int sp = u / LM_SUBS, j = u % LM_SUBS;
        const int len = sp < n_splits ? base + (sp < rem ? 1 : 0) : 0;
        return split_begin(sp) + j * len / LM_SUBS;
    }
};

// Fold of two partial results of one row, (M, S, X, A) <- (M, S, X, A) + (m, s, x, a): the operation by which the units
// of a split are combined, in unit order, starting from (kFloorM, 0, -inf, 0).  Written out operation by operation
// and never contracted, because two kernels must produce the same bits with it.
__device__ __forceinline__ void lm_fold_unit(float &M, float &S, float &X, float &A, float m, float s, float x, float a) {
#pragma clang fp contract(off)
    const float mn = fmaxf(M, m);
    const float f_old = fast_exp2((M - mn) * 1.44269504088896340736f);
    const float f_new = fast_exp2((m - mn) * 1.44269504088896340736f);
    const float s_old = S * f_old, s_new = s * f_new;
    const float a_old = A * f_old, a_new = a * f_new;
    S = s_old + s_new;
    A = a_old + a_new;
    X = fmaxf(X, x);
    M = mn;
}

// Work items are (token block, split) pairs - or, with few rows, (token block, unit) pairs, for which "split" below
// reads "unit" - grouped into super-tiles of tbw token blocks x 32 / tbw splits.  Item v
// belongs to the workgroup v % grid; with a grid of 256 that workgroup sits on XCD v % 8 and holds position
// (v / 8) % 32 of the super-tile that its XCD works on in round v / 256, so the 32 CUs of an XCD run one
// super-tile side by side and fetch 12 distinct slabs per step instead of 64.
// Order of the super-tiles: token-block groups are taken eight at a time, one per XCD, and every XCD keeps its
// token blocks while it walks all split groups: the hidden rows stay in its L2 / the memory-side cache,
// and the eight XCDs stream the same W tiles at the same time, so one fetch from HBM serves them all.  (With
// the token-block group changing at every item each item started on cold hidden rows: 3.5 % slower at
// 32,768 rows.)  The up to seven token-block groups left over are spread over the XCDs split group by split
// group, which is also the whole order for fewer than eight groups.
// Shape of the super-tile: 8 token blocks x 4 splits when that fills the XCDs eight groups at a time (64 token
// blocks or more: every XCD then passes over W half as often; 2 - 3 % faster at 32,768 rows), else 4 x 8.
// Neither the order nor the shape changes any result.  Pairs past the ends of the two ranges are not items.
struct ItemOrder {
    int fine;       // 1: items are (token block, unit) pairs in the plain order described below
    int n_token_blocks, n_cols;  // the two ranges (n_cols: splits, or units)
    SplitPlan plan;
    int tbw, spw;   // token blocks and splits of a super-tile (tbw * spw == 32)
    int sp_groups;  // ceil(n_splits / spw)
    int full;       // token-block groups handled eight at a time
    int rest;       // token-block groups left over (0..7)
    __host__ __device__ ItemOrder(int n_token_blocks_, const SplitPlan &plan_, int fine_) : plan(plan_) {
        fine = fine_;
        n_token_blocks = n_token_blocks_;
        n_cols = fine ? plan.n_splits * LM_SUBS : plan.n_splits;
        tbw = n_token_blocks >= 64 ? 8 : 4;
        spw = 32 / tbw;
        const int tb_groups = (n_token_blocks + tbw - 1) / tbw;
        sp_groups = (n_cols + spw - 1) / spw;
        full = tb_groups / 8 * 8;
        rest = tb_groups - full;
    }
    __host__ __device__ int rounds_full() const { return full / 8 * sp_groups; }
    __host__ __device__ int64_t n_virtual() const {  // item indices in use
        if (fine) return int64_t(n_token_blocks) * ((n_cols + 7) / 8 * 8);
        return (int64_t(rounds_full()) + (rest * sp_groups + 7) / 8) * 256;  // 256 per round
    }
    // Vocabulary tiles [begin, end) of column c.
    __host__ __device__ int col_begin(int c) const {
        return fine ? plan.unit_begin(c) : plan.split_begin(c);
    }
};

// Few rows: item v = ((unit / 8) * n_token_blocks + token block) * 8 + unit % 8, so that unit u is worked on by XCD
// u % 8 for all token blocks at about the same time (its W tiles are fetched from HBM once) and consecutive units
// go to different XCDs.  Empty units are not items.
__device__ __forceinline__ bool lm_decode(int v, const ItemOrder &order, int &tb, int &sp) {
    if (order.fine) {
        const int q = v / 8;
        tb = q % order.n_token_blocks;
        sp = (q / order.n_token_blocks) * 8 + v % 8;
        return sp < order.n_cols && order.col_begin(sp) < order.col_begin(sp + 1);
    }
    const int xcd = v % 8, slot = v / 8;
    const int round = slot / 32, w = slot % 32;
    int tg, sg;
    if (round < order.rounds_full()) {
        tg = (round / order.sp_groups) * 8 + xcd;
        sg = round % order.sp_groups;
    } else {
        const int q = (round - order.rounds_full()) * 8 + xcd;
        const int rest = order.rest > 0 ? order.rest : 1;
        tg = order.full + q % rest;
        sg = q / rest;
    }
    tb = tg * order.tbw + w / order.spw;
    sp = sg * order.spw + w % order.spw;
    return tb < order.n_token_blocks && sp < order.n_cols;
}
// The next item of the workgroup that holds item v: indices advance by the grid size.  >= n_virtual: none.
__device__ __forceinline__ int lm_next_item(int v, int stride, int n_virtual, const ItemOrder &order) {
    int tb, sp;
    do v += stride;
    while (v < n_virtual && !lm_decode(v, order, tb, sp));
    return v;
}

struct Partial {
    float m;   // max logit seen (>= kFloor)
    float s;   // sum of exp(logit - m)
    float xt;  // target logit if this split holds it, else -inf
    float pad; // ENTROPY: sum of x * exp(x - m), else 0
};

// LDS slab: 256 rows x 64 bf16 (128 B per row = eight 16-byte chunks).  A fragment read (ds_read_b128) has
// lane l fetch row l % 32 at logical chunk 2*kk + l / 32.  The chunk index is XOR-swizzled with
// swz(row) = (row >> 1) & 7; measured with a ds_read_b128 micro-benchmark on gfx950 this pattern reads at
// the same rate as a contiguous one, while (row & 7) and an unswizzled slab cost 1.5x and 4.5x.
__device__ __forceinline__ int swz(int row) { return (row >> 1) & 7; }

typedef __attribute__((address_space(3))) void lds_void;

// WIDE: a matrix of 4 GiB or more.  Hidden rows are then addressed relative to the cursor's token block and W rows by
// 64-bit offsets; the ordinary kernel keeps 32-bit offsets from the two base pointers, which is 1 - 2 % faster.
// ENTROPY: also accumulate sum(x * exp(x - max)) per token (one more FMA per logit), from which the fold derives the
// entropy of the row's softmax; it goes out in the fourth field of the partial.
// DLOGITS: the backward's first half instead of the forward.  The same tiles are computed, but each logit x of token n
// goes out as the gradient of that token's log-probability with respect to it, grad[n] * ([v == id_n] - exp(x - lse[n])),
// rounded to bf16, into a [n_rows, vocab] matrix; lse[n] is the row's log-sum-exp as the forward returns it.  No partials,
// no folds; items are (token block, split) pairs.
struct DlogitsArgs {
    const float *lse;    // [n_rows]
    const float *grad;   // [n_rows] upstream gradient of the log-probabilities
    uint16_t *out;       // [n_rows, row_stride] bf16
    int64_t row_stride;  // elements, a multiple of 4 (8-byte stores)
};

template <bool WIDE, bool ENTROPY, bool DLOGITS = false>
__global__ __launch_bounds__(LM_THREADS, 1) void lmhead_partials(
    const uint16_t *__restrict__ hidden, const uint16_t *__restrict__ weight, const int64_t *__restrict__ ids,
    Partial *__restrict__ partials, int n_rows, int hdim, int vocab, int n_token_blocks,
    SplitPlan plan, int n_virtual, int fine, DlogitsArgs dl) {
    extern __shared__ __attribute__((aligned(16))) uint16_t lds[];  // [stage][A = W slab | B = hidden slab]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wave_m = wave >> 1;  // which 128 vocabulary rows of the tile
    const int wave_n = wave & 1;   // which 128 tokens of the block
    const int l32 = lane & 31;
    const int lhalf = lane >> 5;

    // A workgroup walks its items v = blockIdx.x, + gridDim.x, ...: with one workgroup per CU nothing is
    // dispatched between items, and the copies of an item's first slabs are requested while the item before
    // it is still being multiplied.
    const ItemOrder order(n_token_blocks, plan, fine);
    const int stride = gridDim.x;
    const int nk = hdim / LM_BK;
    int v = blockIdx.x, tb, sp;  // sp: the item's column (split, or unit when fine)
    if (!lm_decode(v, order, tb, sp)) v = lm_next_item(v, stride, n_virtual, order);
    if (v >= n_virtual) return;

    float m_run[4], ml2_run[4], s_run[4], xt[4];  // ml2_run = m_run * log2(e), kept so that it is never recomputed
    float a_run[4];                               // ENTROPY: sum of x * exp(x - m_run)
    int target[4];
    float lse2[4], gup[4];                        // DLOGITS: lse * log2(e) and the upstream gradient of the lane's tokens

    // Global -> LDS copies.  One global_load_lds_dwordx4 moves 16 B per lane to LDS base + 16 * lane,
    // i.e. one wavefront fills eight consecutive 128-byte rows (eight full cache lines); instruction j of
    // wavefront w covers rows (4j + w) * 8 .. + 7.  Lane l therefore fetches row (4j + w) * 8 + l / 8 and,
    // because the slab is swizzled, the logical chunk (l % 8) ^ swz(row).  Row offsets are 32-bit byte offsets
    // from a wavefront-uniform base: the matrix itself, or with WIDE the cursor's token block (hidden) and a
    // 64-bit product (W).
    const int cp_row = wave * 8 + (lane >> 3);                 // + 32 * j
    uint32_t hoff[8];                                          // hidden rows of the copy cursor's token block
    int cp_chunk[8];                                           // swz depends on bits 1..3 of the row: on j too
#pragma unroll
    for (int j = 0; j < 8; ++j) cp_chunk[j] = (lane & 7) ^ swz(cp_row + 32 * j);
#define LM_SET_HOFF(tok0_)                                                                                    \
    do {                                                                                                     \
        _Pragma("unroll") for (int j = 0; j < 8; ++j)                                                        \
            hoff[j] = uint32_t(min(cp_row + 32 * j + (WIDE ? 0 : (tok0_)), n_rows - 1 - (WIDE ? (tok0_) : 0))) * row_bytes + cp_chunk[j] * 16u; \
        if (WIDE) hbase = reinterpret_cast<const char *>(hidden) + size_t(tok0_) * row_bytes;                \
    } while (0)
    // W rows of the copy cursor's vocabulary tile: byte offsets from the matrix, computed when the cursor enters a
    // tile, so that a copy costs no vector arithmetic (WIDE computes its 64-bit offsets per copy instead).
    uint32_t woff[8];
#define LM_SET_WOFF(vt_)                                                                                      \
    do {                                                                                                     \
        if constexpr (!WIDE) {                                                                               \
            _Pragma("unroll") for (int j = 0; j < 8; ++j)                                                    \
                woff[j] = uint32_t(min(vt_ * LM_BM + cp_row + 32 * j, vocab - 1)) * row_bytes + cp_chunk[j] * 16u; \
        }                                                                                                    \
    } while (0)
    const uint32_t row_bytes = uint32_t(hdim) * 2u;
    const char *hbase = reinterpret_cast<const char *>(hidden);  // WIDE: first hidden row of the cursor's token block
    LM_SET_HOFF(tb * LM_BN);
    const int wave_lds = __builtin_amdgcn_readfirstlane(wave) * 512;  // bf16 elements: 8 rows of 64
    const char *const wbytes = reinterpret_cast<const char *>(weight);

    // Requests copy c of slab (vt_, kt_) into stage stage_: copies 0..7 fetch the W rows, copies 8..15 the hidden
    // rows.  W first, because its copies take longer (a W tile is streamed once per pass, the hidden rows of the
    // token block come back from cache at every tile) and the first copies of a window have the longest time to
    // land: measured 5 % faster than alternating W and hidden copies, 4 % faster than hidden first.
#define LM_ISSUE_ONE(c_, vt_, kt_, stage_)                                                                   \
    do {                                                                                                     \
        const size_t kb_ = size_t(kt_) * (LM_BK * 2);                                                \
        uint16_t *sa_ = lds + (stage_) * LM_STAGE_ELEMS + wave_lds + ((c_) & 7) * 2048;                        \
        if ((c_) < 8) {                                                                                      \
            if constexpr (WIDE) {                                                                            \
                const uint32_t wrow_ = uint32_t(min((vt_) * LM_BM + cp_row + 32 * (c_), vocab - 1));           \
                const uint64_t woff_ = uint64_t(wrow_) * row_bytes + uint32_t(cp_chunk[(c_) & 7] * 16);        \
                __builtin_amdgcn_global_load_lds(wbytes + kb_ + woff_, (lds_void *)sa_, 16, 0, 0);           \
            } else {                                                                                         \
                __builtin_amdgcn_global_load_lds(wbytes + kb_ + woff[(c_) & 7], (lds_void *)sa_, 16, 0, 0);   \
            }                                                                                                \
        } else {                                                                                             \
            __builtin_amdgcn_global_load_lds(hbase + kb_ + hoff[(c_) & 7], (lds_void *)(sa_ + LM_BM * LM_BK), 16, 0, 0); \
        }                                                                                                    \
    } while (0)

    // Copy cursor: the next slab to request.  It runs up to two slabs ahead of the MFMAs and crosses from an
    // item's last slab into the first slab of the workgroup's next item.  Past the last slab of the last item
    // it stays there (redundant copies into the idle stage), so that every step issues the same copies.
    int v_c = v, vt_c = order.col_begin(sp), vt_end_c = order.col_begin(sp + 1);
    int kt_c = 0;
    LM_SET_WOFF(vt_c);
    // The cursor moves once per slab.  Where to is worked out ahead of the slab's unrolled groups (scalar work, with a
    // search for the workgroup's next item at the end of an item: too long to sit inside the unrolled loop) and
    // committed in group LM_ADV.
    int nx_v = v, nx_vt = vt_c, nx_vt_end = vt_end_c, nx_kt = 0, nx_tb = -1;  // nx_tb >= 0: the token block changes
#define LM_PLAN_CURSOR_MOVE()                                                                                 \
    do {                                                                                                     \
        nx_v = v_c; nx_vt = vt_c; nx_vt_end = vt_end_c; nx_kt = kt_c; nx_tb = -1;                            \
        if (kt_c + 1 < nk) nx_kt = kt_c + 1;                                                                 \
        else if (vt_c + 1 < vt_end_c) { nx_vt = vt_c + 1; nx_kt = 0; }                                       \
        else {                                                                                               \
            const int nv_ = lm_next_item(v_c, stride, n_virtual, order);                                     \
            if (nv_ < n_virtual) {                                                                           \
                int tb_, sp_;                                                                                \
                lm_decode(nv_, order, tb_, sp_);                                                             \
                nx_v = nv_;                                                                                  \
                nx_vt = order.col_begin(sp_);                                                                \
                nx_vt_end = order.col_begin(sp_ + 1);                                                        \
                nx_kt = 0;                                                                                   \
                nx_tb = tb_;                                                                                 \
            }                                                                                                \
        }                                                                                                    \
    } while (0)
#define LM_COMMIT_CURSOR_MOVE()                                                                               \
    do {                                                                                                     \
        const bool new_tile_ = nx_vt != vt_c || nx_tb >= 0;                                                  \
        v_c = nx_v; vt_c = nx_vt; vt_end_c = nx_vt_end; kt_c = nx_kt;                                        \
        if (nx_tb >= 0) LM_SET_HOFF(nx_tb * LM_BN);                                                          \
        if (new_tile_) LM_SET_WOFF(vt_c);                                                                    \
    } while (0)
    // Fragment addresses.  swz() of a fragment row does not depend on the 32-row block (t * 32 and wave * 128 do not
    // touch bits 1..3), so block t of an operand sits t * 4096 bytes behind block 0 and only the k-step changes the
    // chunk: one LDS pointer per (k-step, operand) into the stage in use, kept in registers, with the block as an
    // immediate offset of the read.  Nothing is computed per read; the eight pointers move to the other stage once
    // per slab (stage_step: + one stage, then - one stage, ...).
    typedef __attribute__((address_space(3))) const unsigned char lds_cbyte;
    typedef __attribute__((address_space(3))) const bf16x8 lds_frag;
    lds_cbyte *const lds3 = (lds_cbyte *)lds;
    lds_cbyte *pa[4], *pb[4];
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
        const int chunk = ((kk * 2 + lhalf) ^ swz(l32)) << 4;
        pa[kk] = lds3 + (wave_m * 128 + l32) * (LM_BK * 2) + chunk;
        pb[kk] = lds3 + (LM_BM + wave_n * 128 + l32) * (LM_BK * 2) + chunk;
    }
    int stage_step = LM_STAGE_ELEMS * 2;  // bytes from the stage in use to the other one
#define LM_FRAG(ptr_, t_) (*(lds_frag *)((ptr_) + (t_) * (32 * LM_BK * 2)))

    // Software pipeline, per slab s (stage s & 1) in 32 groups of two MFMAs:
    //   groups  0..7   request copies 8..15 of slab s + 1 (other stage);
    //   group   24     waits for slab s + 1 (vmcnt(0)) and for this wavefront's last fragment reads of slab s
    //                  (lgkmcnt(0)), then s_barrier: slab s + 1 is complete in LDS and nobody reads slab s any more;
    //   groups 24..27  read the k-step-0 fragments of slab s + 1, so that the next slab starts without waiting
    //                  for LDS;
    //   groups 24..31  request copies 0..7 of slab s + 2 into the stage slab s has just left.
    // An MFMA blocks the issue port for its 8 passes, so a read that follows its consumer's predecessors in
    // program order would issue too late to hide its latency: the order below is pinned with sched_barrier.
#pragma unroll
    for (int c = 0; c < 16; ++c) LM_ISSUE_ONE(c, vt_c, kt_c, 0);
    LM_PLAN_CURSOR_MOVE();
    LM_COMMIT_CURSOR_MOVE();
#pragma unroll
    for (int c = 0; c < LM_FIRST; ++c) LM_ISSUE_ONE(c, vt_c, kt_c, 1);  // the rest of slab 1 follows in the groups of slab 0
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(LM_FIRST) : "memory");  // copies complete in order: slab 0 is in
    bf16x8 fa[2][4], fb[2][4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        fa[0][t] = LM_FRAG(pa[0], t);
        fb[0][t] = LM_FRAG(pb[0], t);
    }

    int stage = 0;
    float *const xch = reinterpret_cast<float *>(lds + LM_STAGES * LM_STAGE_ELEMS);  // [wave_n][tn][32][4]
    float *const split_acc = xch + LM_XCH_BYTES / 4;                                  // same shape
    const bool folder = wave_m == 0 && lhalf == 0;  // the lanes that end up with a token's folded partial
    for (;;) {  // items of this workgroup; v is a valid item here
    lm_decode(v, order, tb, sp);
    const int tok0 = tb * LM_BN;
    // This lane's four tokens (one per 32-column block of the wave tile) and their targets.
#pragma unroll
    for (int tn = 0; tn < 4; ++tn) {
        const int n = tok0 + wave_n * 128 + tn * 32 + l32;
        int64_t id = -1;
        if (n < n_rows) id = ids[n];
        target[tn] = (id >= 0 && id < vocab) ? int(id) : -1;
        if constexpr (DLOGITS) {
            lse2[tn] = n < n_rows ? dl.lse[n] * kLog2e : 0.0f;
            gup[tn] = n < n_rows ? dl.grad[n] : 0.0f;
        }
        if (!DLOGITS && !fine && folder) {  // the split's running partial starts empty
            float *p = split_acc + ((wave_n * 4 + tn) * 32 + l32) * 4;
            p[0] = kFloor;
            p[1] = 0.0f;
            p[2] = -__builtin_inff();
            p[3] = 0.0f;
        }
    }
    // The units of the item: its own when the item is a unit, else those of its split, in order.
    const int u_first = fine ? sp : sp * LM_SUBS, u_last = fine ? sp + 1 : (sp + 1) * LM_SUBS;
    for (int u = u_first; u < u_last; ++u) {
    const int vt_begin = plan.unit_begin(u);
    const int vt_end = plan.unit_begin(u + 1);
    if (vt_begin == vt_end) continue;  // (workgroup-uniform) a split of fewer than LM_SUBS tiles has empty units
#pragma unroll
    for (int tn = 0; tn < 4; ++tn) {
        m_run[tn] = kFloor;
        ml2_run[tn] = kFloor * kLog2e;
        s_run[tn] = 0.0f;
        a_run[tn] = 0.0f;
        xt[tn] = -__builtin_inff();
    }
    for (int vt = vt_begin; vt < vt_end; ++vt) {
        f32x16 acc[4][4];
#pragma unroll
        for (int tm = 0; tm < 4; ++tm)
#pragma unroll
            for (int tn = 0; tn < 4; ++tn)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[tm][tn][r] = 0.0f;

        // Per group: first MFMA, the group's fragment reads, second MFMA, the group's copy: each MFMA covers the
        // issue of at most two other instructions.
        for (int kt = 0; kt < nk; ++kt) {
            LM_PLAN_CURSOR_MOVE();
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int g = 0; g < 32; ++g) {
                const int kk = g >> 3, sub = g & 7;  // 8 groups of 2 MFMAs per k-step
                {
                    const int m = sub * 2, tm = m >> 2, tn = m & 3;
                    acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[kk & 1][tm], fb[kk & 1][tn], acc[tm][tn], 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
                if (kk < 3 && sub < 4) {  // both reads early in the k-step: they have returned when it ends
                    fa[(kk + 1) & 1][sub] = LM_FRAG(pa[kk + 1], sub);
                    fb[(kk + 1) & 1][sub] = LM_FRAG(pb[kk + 1], sub);
                }
                if (g == LM_BAR) {
                    // Builtins rather than inline asm: the compiler's own wait-count bookkeeping sees them, so it
                    // does not add a conservative lgkmcnt(0) behind the fresh reads that follow.
                    __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
                    __builtin_amdgcn_s_barrier();
                    // every read of this slab has been issued: the pointers move to the stage of the next slab
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        pa[q] += stage_step;
                        pb[q] += stage_step;
                    }
                    stage_step = -stage_step;
                }
                if (g >= LM_BAR && g < LM_BAR + 4) {
                    fa[0][g - LM_BAR] = LM_FRAG(pa[0], g - LM_BAR);
                    fb[0][g - LM_BAR] = LM_FRAG(pb[0], g - LM_BAR);
                }
                __builtin_amdgcn_sched_barrier(0);
                {
                    const int m = sub * 2 + 1, tm = m >> 2, tn = m & 3;
                    acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[kk & 1][tm], fb[kk & 1][tn], acc[tm][tn], 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
                {
                    // copies of this group: behind the barrier they belong to the slab whose window has just opened
                    // (the cursor has moved on to it) and go to the stage that the barrier has freed
                    if (g == LM_ADV) LM_COMMIT_CURSOR_MOVE();
                    const int c0 = kCopyTable.at[g];  // compile-time: g is unrolled
                    if (c0 >= 0) LM_ISSUE_ONE(c0, vt_c, kt_c, g >= LM_BAR ? stage : stage ^ 1);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            stage ^= 1;
        }

        // ---- the logits of this vocabulary tile are complete: fold them into the running state ----
        // Vocabulary row of acc[tm][tn][r]: vrow0 + tm*32 + (r/4)*8 + r%4.
        const int vrow0 = vt * LM_BM + wave_m * 128 + lhalf * 4;
        const int limit = vocab - vrow0;  // rows at offset >= limit lie past the vocabulary (last tile only)
#pragma unroll
        for (int tn = 0; tn < 4; ++tn) {
#pragma clang fp contract(off)  // (mn * log2e feeds a difference: as part of an FMA it would not cancel at the floor)
            // keep the four token blocks apart: only 64 accumulators are live in VGPRs at a time
            __builtin_amdgcn_sched_barrier(0);
            const int d = target[tn] - (vt * LM_BM + wave_m * 128);
            const bool mine = d >= 0 && d < 128 && ((d >> 2) & 1) == lhalf;
            const int want = mine ? (((d >> 5) << 4) | ((d & 31) >> 3 << 2) | (d & 3)) : -1;  // tm*16 + r
            if constexpr (DLOGITS) {
                // four consecutive vocabulary rows of one token per store: 8 bytes at out[n, vrow0 + tm*32 + q*8 ..]
                const int n = tok0 + wave_n * 128 + tn * 32 + l32;
                uint16_t *const orow = dl.out + size_t(n < n_rows ? n : 0) * size_t(dl.row_stride) + vrow0;
                const float g = gup[tn], l2 = lse2[tn];
#pragma unroll
                for (int tm = 0; tm < 4; ++tm)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        union { __bf16 h[4]; uint2 u; } pk;
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            const float pr = fast_exp2(fmaf(acc[tm][tn][q * 4 + j], kLog2e, -l2));
                            const float onehot = want == tm * 16 + q * 4 + j ? g : 0.0f;
                            pk.h[j] = (__bf16)fmaf(-g, pr, onehot);
                        }
                        const int off = tm * 32 + q * 8;
                        if (n < n_rows) {
                            if (off + 3 < limit) {
                                *reinterpret_cast<uint2 *>(orow + off) = pk.u;
                            } else {
#pragma unroll
                                for (int j = 0; j < 4; ++j)
                                    if (off + j < limit) orow[off + j] = reinterpret_cast<const uint16_t *>(pk.h)[j];
                            }
                        }
                    }
                continue;
            }
            float mn = m_run[tn];
            float part[4], parta[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            // Wavefront-uniform choice: almost every tile lies inside the vocabulary and holds no lane's target,
            // and then needs neither the bounds select nor the capture compare per logit.
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
                    if constexpr (ENTROPY) {  // logits inside the vocabulary are finite: no 0 * inf here
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
                        if constexpr (ENTROPY) xe[r] = e[r] == 0.0f ? 0.0f : x * e[r];  // rows past the vocabulary: 0, not 0 * -inf
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
            // difference of the two stored products: recomputing m_run * log2e here could be fused into an
            // FMA against ml2n and return the rounding residue of a 1e30-sized product instead of 0
            const float rescale = fast_exp2(ml2_run[tn] - ml2n);
            s_run[tn] = fmaf(s_run[tn], rescale, (part[0] + part[1]) + (part[2] + part[3]));
            if constexpr (ENTROPY) a_run[tn] = fmaf(a_run[tn], rescale, (parta[0] + parta[1]) + (parta[2] + parta[3]));
            m_run[tn] = mn;
            ml2_run[tn] = ml2n;
        }
        __builtin_amdgcn_sched_barrier(0);
    }

    if constexpr (!DLOGITS) {
    // ---- fold the two lane halves (rows 4..7 of each 8-row group live in lanes 32..63) ----
#pragma unroll
    for (int tn = 0; tn < 4; ++tn) {
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
    // ---- fold the two vocabulary halves of the tile through LDS (upper half -> lower half) ----
    // The exchange area lies behind the two stages, which already receive the slabs of the next unit or item.
    // One barrier is enough: the area is written again only after another unit's slabs, each with a barrier.
    if (wave_m == 1 && lhalf == 0) {
#pragma unroll
        for (int tn = 0; tn < 4; ++tn) {
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
        for (int tn = 0; tn < 4; ++tn) {
            const float *p = xch + ((wave_n * 4 + tn) * 32 + l32) * 4;
            const float om = p[0], os = p[1], ox = p[2];
            const float mm = fmaxf(m_run[tn], om);
            const float f_own = fast_exp2((m_run[tn] - mm) * kLog2e), f_other = fast_exp2((om - mm) * kLog2e);
            const float s = s_run[tn] * f_own + os * f_other;
            float a = 0.0f;
            if constexpr (ENTROPY) a = a_run[tn] * f_own + p[3] * f_other;
            const float x = fmaxf(xt[tn], ox);
            const int n = tok0 + wave_n * 128 + tn * 32 + l32;
            if (fine) {  // the unit's partial goes out as it is; the second kernel folds the units
                if (n < n_rows) {
                    Partial out;
                    out.m = mm;
                    out.s = s;
                    out.xt = x;
                    out.pad = a;
                    partials[size_t(u) * n_rows + n] = out;
                }
            } else {
                float *q = split_acc + ((wave_n * 4 + tn) * 32 + l32) * 4;
                float M = q[0], S = q[1], X = q[2], A = q[3];
                lm_fold_unit(M, S, X, A, mm, s, x, a);
                q[0] = M;
                q[1] = S;
                q[2] = X;
                q[3] = A;
            }
        }
    }
    }  // !DLOGITS
    }  // units
    if (!DLOGITS && !fine && folder) {
#pragma unroll
        for (int tn = 0; tn < 4; ++tn) {
            const float *q = split_acc + ((wave_n * 4 + tn) * 32 + l32) * 4;
            const int n = tok0 + wave_n * 128 + tn * 32 + l32;
            if (n < n_rows) {
                Partial out;
                out.m = q[0];
                out.s = q[1];
                out.xt = q[2];
                out.pad = q[3];
                partials[size_t(sp) * n_rows + n] = out;
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

#include "ka_lmhead_narrow.h"

namespace ka {
namespace {

// The fold of a row's split partials, in split order, and the two results.  get(sp) returns the partial of split sp.
// Written out operation by operation (no contraction): whoever produced the split partials, the bits are the same.
template <typename Get>
__device__ __forceinline__ void lm_finish_row(Get get, int n_splits, int64_t id, int vocab, float *out_slot, float *entropy_slot,
                                              float *lse_slot) {
#pragma clang fp contract(off)
    float mm = kFloor;
    for (int sp = 0; sp < n_splits; ++sp) mm = fmaxf(mm, get(sp).m);
    float s = 0.0f, a = 0.0f, x = -__builtin_inff();
    for (int sp = 0; sp < n_splits; ++sp) {  // fixed split order
        const Partial p = get(sp);
        const float f = fast_exp2((p.m - mm) * kLog2e);
        const float ts = p.s * f, ta = p.pad * f;
        s = s + ts;
        a = a + ta;
        x = fmaxf(x, p.xt);
    }
    const double lse = double(mm) + log2(double(s)) * kLn2;
    if (entropy_slot != nullptr) *entropy_slot = float(lse - double(a) / double(s));  // -sum p log p = lse - sum p x
    if (lse_slot != nullptr) *lse_slot = float(lse);
    if (id < 0 || id >= vocab) {
        *out_slot = __builtin_nanf("");
        return;
    }
    *out_slot = float(double(x) - lse);
}

// One thread per row; the kernel before it has folded the units of every split.
__global__ __launch_bounds__(256) void lmhead_combine(const Partial *__restrict__ partials,
                                                      const int64_t *__restrict__ ids, float *__restrict__ out,
                                                      float *__restrict__ entropy, float *__restrict__ lse, int n_rows,
                                                      int vocab, int n_splits) {
    const int n = blockIdx.x * blockDim.x + threadIdx.x;
    if (n >= n_rows) return;
    lm_finish_row([&](int sp) { return partials[size_t(sp) * n_rows + n]; }, n_splits, ids[n], vocab, out + n,
                  entropy != nullptr ? entropy + n : nullptr, lse != nullptr ? lse + n : nullptr);
}

// Few rows: the kernel before it has written one partial per unit.  One wavefront per row: lane l folds the units of
// the splits l, l + 64, ... in unit order (the same operations as the other kernel performs in place) into LDS, then
// the splits are folded as above.
constexpr int LM_FINE_MAX_SPLITS = 256;
__global__ __launch_bounds__(256) void lmhead_combine_units(const Partial *__restrict__ partials,
                                                            const int64_t *__restrict__ ids, float *__restrict__ out,
                                                            float *__restrict__ entropy, float *__restrict__ lse,
                                                            int n_rows, int vocab, SplitPlan plan) {
    __shared__ Partial folded[4][LM_FINE_MAX_SPLITS];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int n = blockIdx.x * 4 + wave;
    if (n >= n_rows) return;  // wavefront-uniform; nothing below synchronises across wavefronts
    const int n_splits = plan.n_splits;
    for (int sp = lane; sp < n_splits; sp += kWave) {
        float M = kFloor, S = 0.0f, X = -__builtin_inff(), A = 0.0f;
        for (int j = 0; j < LM_SUBS; ++j) {
            const int u = sp * LM_SUBS + j;
            if (plan.unit_begin(u) == plan.unit_begin(u + 1)) continue;  // empty unit
            const Partial p = partials[size_t(u) * n_rows + n];
            lm_fold_unit(M, S, X, A, p.m, p.s, p.xt, p.pad);
        }
        Partial q;
        q.m = M;
        q.s = S;
        q.xt = X;
        q.pad = A;
        folded[wave][sp] = q;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if (lane == 0)
        lm_finish_row([&](int sp) { return folded[wave][sp]; }, n_splits, ids[n], vocab, out + n,
                      entropy != nullptr ? entropy + n : nullptr, lse != nullptr ? lse + n : nullptr);
}

inline int splits_for(int64_t vocab) {
    const int64_t n_vtiles = (vocab + LM_BM - 1) / LM_BM;
    return lm_n_splits(int(n_vtiles));
}

// Items are units instead of whole splits when whole splits would leave CUs without an item (the kernel runs one
// workgroup on each of 256 CUs).  The choice changes the schedule and the size of the workspace, not a result bit.
constexpr int LM_RESIDENT = 256;
// Up to this many rows a call runs the kernel of ka_lmhead_narrow.h (64 tokens per workgroup up to 64 rows, 128 above).
// (Measured at V = 128,256, H = 4096: 64 rows 0.27 -> 0.20 ms, 128 rows 0.27 -> 0.21 ms; 256 rows as two 128-token blocks
// 0.35 ms against 0.30 ms for the 256-token kernel, so the limit stays at one 128-token block.)
constexpr int LN_MAX_ROWS = 128;
inline bool units_as_items(int64_t n_rows, int64_t vocab) {
    const int64_t n_token_blocks = (n_rows + LM_BN - 1) / LM_BN;
    const int n_splits = splits_for(vocab);
    return n_token_blocks * n_splits < LM_RESIDENT && n_splits <= LM_FINE_MAX_SPLITS;
}

}  // namespace
}  // namespace ka

KA_EXPORT size_t ka_lmhead_workspace_bytes(int64_t n_rows, int64_t hidden_dim, int64_t vocab) {
    (void)hidden_dim;
    if (n_rows <= 0 || vocab <= 0) return 0;
    const size_t per_row = size_t(ka::splits_for(vocab)) * (ka::units_as_items(n_rows, vocab) ? ka::LM_SUBS : 1);
    return per_row * size_t(n_rows) * sizeof(ka::Partial);
}

namespace ka {
namespace {

// Scratch of ka_lmhead_logprob_bf16_noalloc: the partials of one call live here instead of in a caller's workspace.
// Every GPU the library runs on holds its own copy of the array until the process ends.  In host code the array's
// name is only a handle for hipGetSymbolAddress: kernels are given the device address looked up below.
constexpr size_t LM_STATIC_SCRATCH_BYTES = KA_LMHEAD_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char lm_static_scratch[LM_STATIC_SCRATCH_BYTES];

// What the launch needs to know about a device, looked up once per device with that device current.
struct LmDevice {
    bool ready = false;          // cus is valid and both kernels have their LDS size reserved on this device
    bool scratch_ready = false;  // scratch is valid
    int cus = 0;
    void *scratch = nullptr;     // device address of this device's lm_static_scratch
};
constexpr int LM_MAX_DEVICES = 64;
LmDevice g_lm_device[LM_MAX_DEVICES];
std::mutex g_lm_device_mutex;

// Fills `out` with the current device's record (a copy: the table is only touched under the mutex).
int lm_current_device(bool need_scratch, LmDevice &out) {
    int device = 0;
    hipError_t rc = hipGetDevice(&device);
    if (rc != hipSuccess) return check_hip(rc, "lmhead: hipGetDevice");
    if (device < 0 || device >= LM_MAX_DEVICES) return fail(KA_ERR_UNSUPPORTED, "lmhead: device index %d", device);
    std::lock_guard<std::mutex> lock(g_lm_device_mutex);
    LmDevice &d = g_lm_device[device];
    if (!d.ready) {
        int cus = 0;
        rc = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device);
        if (rc != hipSuccess) return check_hip(rc, "lmhead: querying the CU count");
        // the attribute belongs to the device, so it is set once per device and not once per process
        const void *kernels[6] = {reinterpret_cast<const void *>(lmhead_partials<false, false>),
                                  reinterpret_cast<const void *>(lmhead_partials<true, false>),
                                  reinterpret_cast<const void *>(lmhead_partials<false, true>),
                                  reinterpret_cast<const void *>(lmhead_partials<true, true>),
                                  reinterpret_cast<const void *>(lmhead_partials<false, false, true>),
                                  reinterpret_cast<const void *>(lmhead_partials<true, false, true>)};
        for (int k = 0; k < 6 && rc == hipSuccess; ++k)
            rc = hipFuncSetAttribute(kernels[k], hipFuncAttributeMaxDynamicSharedMemorySize, LM_LDS_BYTES);
        if (rc == hipSuccess)
            rc = hipFuncSetAttribute(reinterpret_cast<const void *>(lmhead_partials_narrow<1, false>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, ln_lds_bytes<1>());
        if (rc == hipSuccess)
            rc = hipFuncSetAttribute(reinterpret_cast<const void *>(lmhead_partials_narrow<1, true>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, ln_lds_bytes<1>());
        if (rc == hipSuccess)
            rc = hipFuncSetAttribute(reinterpret_cast<const void *>(lmhead_partials_narrow<2, false>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, ln_lds_bytes<2>());
        if (rc == hipSuccess)
            rc = hipFuncSetAttribute(reinterpret_cast<const void *>(lmhead_partials_narrow<2, true>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, ln_lds_bytes<2>());
        if (rc != hipSuccess) return check_hip(rc, "lmhead: reserving LDS for the kernels");
        d.cus = cus;
        d.ready = true;
    }
    if (need_scratch && !d.scratch_ready) {
        void *ptr = nullptr;
        rc = hipGetSymbolAddress(&ptr, HIP_SYMBOL(lm_static_scratch));
        if (rc != hipSuccess || ptr == nullptr)
            return check_hip(rc != hipSuccess ? rc : hipErrorInvalidSymbol, "lmhead: address of the static scratch array");
        d.scratch = ptr;
        d.scratch_ready = true;
    }
    out = d;
    return KA_OK;
}

// Argument checks shared by the two entry points (everything except the workspace).
int lm_check_args(const void *hidden, const void *weight, const int64_t *ids, const float *out, int64_t n_rows,
                  int64_t hidden_dim, int64_t vocab) {
    if (hidden == nullptr || weight == nullptr || ids == nullptr || out == nullptr)
        return fail(KA_ERR_BAD_ARG, "lmhead: null hidden / weight / ids / out pointer");
    if (hidden_dim < 8 || vocab < 1) return fail(KA_ERR_BAD_ARG, "lmhead: hidden_dim %lld, vocab %lld", (long long)hidden_dim, (long long)vocab);
    if (hidden_dim % LM_BK != 0)
        return fail(KA_ERR_UNSUPPORTED, "lmhead: hidden_dim %lld is not a multiple of %d", (long long)hidden_dim, LM_BK);
    if (reinterpret_cast<uintptr_t>(hidden) % 16 != 0 || reinterpret_cast<uintptr_t>(weight) % 16 != 0)
        return fail(KA_ERR_UNSUPPORTED, "lmhead: hidden and weight must be 16-byte aligned");
    if (n_rows >= (int64_t(1) << 31) || vocab >= (int64_t(1) << 31) || hidden_dim >= (int64_t(1) << 31))
        return fail(KA_ERR_UNSUPPORTED, "lmhead: a dimension does not fit 31 bits");
    return KA_OK;
}

// Enqueues the two kernels; `partials` holds ka_lmhead_workspace_bytes(n_rows, ., vocab) bytes of device memory.
int lm_launch(const LmDevice &dev, const void *hidden, const void *weight, const int64_t *ids, float *out,
              float *entropy, float *lse, int64_t n_rows, int64_t hidden_dim, int64_t vocab, Partial *partials, hipStream_t stream) {
    const int n_vtiles = int((vocab + LM_BM - 1) / LM_BM);
    const int n_splits = splits_for(vocab);
    const int n_token_blocks = int((n_rows + LM_BN - 1) / LM_BN);
    const int fine = units_as_items(n_rows, vocab) ? 1 : 0;
    const SplitPlan plan(n_vtiles, n_splits);
    const int64_t n_virtual = ItemOrder(n_token_blocks, plan, fine).n_virtual();
    if (n_virtual >= (int64_t(1) << 30)) return fail(KA_ERR_UNSUPPORTED, "lmhead: too many work items");
    // One workgroup per CU (a workgroup takes a CU's LDS and registers); each walks its items.  256 workgroups
    // keep item v on XCD v % 8 and at one position of its super-tiles.
    const int64_t resident = dev.cus >= LM_RESIDENT ? LM_RESIDENT : (dev.cus >= 8 ? dev.cus / 8 * 8 : 8);
    const int64_t grid = n_virtual < resident ? n_virtual : resident;
    const bool wide = n_rows * hidden_dim * 2 >= (int64_t(1) << 32) || vocab * hidden_dim * 2 >= (int64_t(1) << 32);
    if (fine && !wide && n_rows <= LN_MAX_ROWS) {
        // Few rows: the kernel with 64- or 128-token workgroups and three stages of slabs (ka_lmhead_narrow.h).
        const int tn = n_rows <= 64 ? 1 : 2;
        const int ntb = int((n_rows + 64 * tn - 1) / (64 * tn));
        const int64_t nvirt = ItemOrder(ntb, plan, 1).n_virtual();
        const int64_t g = nvirt < resident ? nvirt : resident;
        auto go = [&](auto kernel, int lds_bytes) {
            hipLaunchKernelGGL(kernel, dim3(unsigned(g)), dim3(LM_THREADS), lds_bytes, stream,
                               static_cast<const uint16_t *>(hidden), static_cast<const uint16_t *>(weight), ids, partials,
                               int(n_rows), int(hidden_dim), int(vocab), ntb, plan, int(nvirt));
        };
        if (tn == 1) {
            if (entropy != nullptr) go(lmhead_partials_narrow<1, true>, ln_lds_bytes<1>());
            else go(lmhead_partials_narrow<1, false>, ln_lds_bytes<1>());
        } else {
            if (entropy != nullptr) go(lmhead_partials_narrow<2, true>, ln_lds_bytes<2>());
            else go(lmhead_partials_narrow<2, false>, ln_lds_bytes<2>());
        }
        const int rcn = check_hip(hipGetLastError(), "lmhead partials launch (few rows)");
        if (rcn != KA_OK) return rcn;
        hipLaunchKernelGGL(lmhead_combine_units, dim3(unsigned((n_rows + 3) / 4)), dim3(256), 0, stream, partials, ids,
                           out, entropy, lse, int(n_rows), int(vocab), plan);
        return check_hip(hipGetLastError(), "lmhead combine launch");
    }
    auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, dim3(unsigned(grid)), dim3(LM_THREADS), LM_LDS_BYTES, stream,
                           static_cast<const uint16_t *>(hidden), static_cast<const uint16_t *>(weight), ids, partials,
                           int(n_rows), int(hidden_dim), int(vocab), n_token_blocks, plan, int(n_virtual), fine, DlogitsArgs{});
    };
    if (entropy != nullptr) {
        if (wide) launch(lmhead_partials<true, true>);
        else launch(lmhead_partials<false, true>);
    } else {
        if (wide) launch(lmhead_partials<true, false>);
        else launch(lmhead_partials<false, false>);
    }
    int rc = check_hip(hipGetLastError(), "lmhead partials launch");
    if (rc != KA_OK) return rc;
    if (fine)
        hipLaunchKernelGGL(lmhead_combine_units, dim3(unsigned((n_rows + 3) / 4)), dim3(256), 0, stream, partials, ids,
                           out, entropy, lse, int(n_rows), int(vocab), plan);
    else
        hipLaunchKernelGGL(lmhead_combine, dim3(unsigned((n_rows + 255) / 256)), dim3(256), 0, stream, partials, ids,
                           out, entropy, lse, int(n_rows), int(vocab), n_splits);
    return check_hip(hipGetLastError(), "lmhead combine launch");
}

// Everything the workspace entry points share.
int lm_with_workspace(const void *hidden, const void *weight, const int64_t *ids, float *out, float *entropy, float *lse,
                      int64_t n_rows, int64_t hidden_dim, int64_t vocab, void *workspace, size_t workspace_bytes,
                      void *hip_stream) {
    if (n_rows < 0) return fail(KA_ERR_BAD_ARG, "lmhead: n_rows %lld < 0", (long long)n_rows);
    if (n_rows == 0) return KA_OK;
    int rc = lm_check_args(hidden, weight, ids, out, n_rows, hidden_dim, vocab);
    if (rc != KA_OK) return rc;
    const size_t need = ka_lmhead_workspace_bytes(n_rows, hidden_dim, vocab);
    if (workspace == nullptr || workspace_bytes < need || reinterpret_cast<uintptr_t>(workspace) % 16 != 0)
        return fail(KA_ERR_WORKSPACE, "lmhead: workspace of %zu B (16-byte aligned) needed, got %zu B", need, workspace_bytes);
    LmDevice dev;
    rc = lm_current_device(false, dev);
    if (rc != KA_OK) return rc;
    return lm_launch(dev, hidden, weight, ids, out, entropy, lse, n_rows, hidden_dim, vocab, static_cast<Partial *>(workspace),
                     static_cast<hipStream_t>(hip_stream));
}

}  // namespace
}  // namespace ka

KA_EXPORT int ka_lmhead_logprob_bf16(const void *hidden, const void *weight, const int64_t *ids, float *out,
                                     int64_t n_rows, int64_t hidden_dim, int64_t vocab, void *workspace,
                                     size_t workspace_bytes, void *hip_stream) {
    return ka::lm_with_workspace(hidden, weight, ids, out, nullptr, nullptr, n_rows, hidden_dim, vocab, workspace, workspace_bytes,
                                 hip_stream);
}

KA_EXPORT int ka_lmhead_logprob_entropy_bf16(const void *hidden, const void *weight, const int64_t *ids, float *out,
                                             float *entropy, int64_t n_rows, int64_t hidden_dim, int64_t vocab,
                                             void *workspace, size_t workspace_bytes, void *hip_stream) {
    if (entropy == nullptr && n_rows > 0) return ka::fail(KA_ERR_BAD_ARG, "lmhead: null entropy pointer");
    return ka::lm_with_workspace(hidden, weight, ids, out, entropy, nullptr, n_rows, hidden_dim, vocab, workspace, workspace_bytes,
                                 hip_stream);
}

KA_EXPORT int ka_lmhead_logprob_lse_bf16(const void *hidden, const void *weight, const int64_t *ids, float *out,
                                         float *lse, int64_t n_rows, int64_t hidden_dim, int64_t vocab, void *workspace,
                                         size_t workspace_bytes, void *hip_stream) {
    if (lse == nullptr && n_rows > 0) return ka::fail(KA_ERR_BAD_ARG, "lmhead: null lse pointer");
    return ka::lm_with_workspace(hidden, weight, ids, out, nullptr, lse, n_rows, hidden_dim, vocab, workspace, workspace_bytes,
                                 hip_stream);
}

KA_EXPORT int ka_lmhead_dlogits_bf16(const void *hidden, const void *weight, const int64_t *ids, const float *lse,
                                     const float *grad_logprob, void *dlogits, int64_t dlogits_row_stride, int64_t n_rows,
                                     int64_t hidden_dim, int64_t vocab, void *hip_stream) {
    using namespace ka;
    if (n_rows < 0) return fail(KA_ERR_BAD_ARG, "lmhead dlogits: n_rows %lld < 0", (long long)n_rows);
    if (n_rows == 0) return KA_OK;
    if (lse == nullptr || grad_logprob == nullptr || dlogits == nullptr)
        return fail(KA_ERR_BAD_ARG, "lmhead dlogits: null lse / grad_logprob / dlogits pointer");
    int rc = lm_check_args(hidden, weight, ids, lse, n_rows, hidden_dim, vocab);
    if (rc != KA_OK) return rc;
    if (dlogits_row_stride < vocab || dlogits_row_stride % 4 != 0 || reinterpret_cast<uintptr_t>(dlogits) % 8 != 0)
        return fail(KA_ERR_BAD_ARG, "lmhead dlogits: the gradient matrix must be 8-byte aligned with a row stride >= vocab that "
                                    "is a multiple of 4 (got %lld)", (long long)dlogits_row_stride);
    LmDevice dev;
    rc = lm_current_device(false, dev);
    if (rc != KA_OK) return rc;
    const int n_vtiles = int((vocab + LM_BM - 1) / LM_BM);
    const SplitPlan plan(n_vtiles, splits_for(vocab));
    const int n_token_blocks = int((n_rows + LM_BN - 1) / LM_BN);
    const int64_t n_virtual = ItemOrder(n_token_blocks, plan, 0).n_virtual();
    if (n_virtual >= (int64_t(1) << 30)) return fail(KA_ERR_UNSUPPORTED, "lmhead dlogits: too many work items");
    const int64_t resident = dev.cus >= LM_RESIDENT ? LM_RESIDENT : (dev.cus >= 8 ? dev.cus / 8 * 8 : 8);
    const int64_t grid = n_virtual < resident ? n_virtual : resident;
    const bool wide = n_rows * hidden_dim * 2 >= (int64_t(1) << 32) || vocab * hidden_dim * 2 >= (int64_t(1) << 32);
    const DlogitsArgs dl{lse, grad_logprob, static_cast<uint16_t *>(dlogits), dlogits_row_stride};
    auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, dim3(unsigned(grid)), dim3(LM_THREADS), LM_LDS_BYTES, static_cast<hipStream_t>(hip_stream),
                           static_cast<const uint16_t *>(hidden), static_cast<const uint16_t *>(weight), ids,
                           static_cast<Partial *>(nullptr), int(n_rows), int(hidden_dim), int(vocab), n_token_blocks, plan,
                           int(n_virtual), 0, dl);
    };
    if (wide) launch(lmhead_partials<true, false, true>);
    else launch(lmhead_partials<false, false, true>);
    return check_hip(hipGetLastError(), "lmhead dlogits launch");
}

KA_EXPORT int ka_lmhead_logprob_bf16_noalloc(const void *hidden, const void *weight, const int64_t *ids, float *out,
                                             int64_t n_rows, int64_t hidden_dim, int64_t vocab, void *hip_stream) {
    using namespace ka;
    if (n_rows < 0) return fail(KA_ERR_BAD_ARG, "lmhead: n_rows %lld < 0", (long long)n_rows);
    if (n_rows == 0) return KA_OK;
    int rc = lm_check_args(hidden, weight, ids, out, n_rows, hidden_dim, vocab);
    if (rc != KA_OK) return rc;
    const size_t need = ka_lmhead_workspace_bytes(n_rows, hidden_dim, vocab);
    if (need > LM_STATIC_SCRATCH_BYTES)
        return fail(KA_ERR_WORKSPACE,
                    "lmhead (noalloc): %lld rows x vocab %lld need %zu B of partials, the static scratch holds %zu B; "
                    "pass fewer rows per call or use ka_lmhead_logprob_bf16 with a workspace",
                    (long long)n_rows, (long long)vocab, need, LM_STATIC_SCRATCH_BYTES);
    LmDevice dev;
    rc = lm_current_device(true, dev);
    if (rc != KA_OK) return rc;
    // Nothing in the scratch has to start at zero: every partial the fold reads is written by this call's first kernel.
    return lm_launch(dev, hidden, weight, ids, out, nullptr, nullptr, n_rows, hidden_dim, vocab, static_cast<Partial *>(dev.scratch),
                     static_cast<hipStream_t>(hip_stream));
}

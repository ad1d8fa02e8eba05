/*
 * ka_oracle.c — exactly specified CPU restatement of the fused sampling operator.
 *
 * TEST INFRASTRUCTURE ONLY: built into oracle/_build/libka_oracle.so and loaded by
 * tests/, __graft_entry__.smoke() and bench.py's checker.  The product library
 * neither links nor calls it.
 *
 * What it restates (reference file:line):
 *   - temperature in the logits' own dtype: rl_engine/kernels/sampling.py:43-45 and
 *     benchmarks/benchmark_sampling.py:16-17  (y = x / T, rounded to the dtype);
 *   - top-k with ties kept: rl_engine/kernels/sampling.py:83-86 and
 *     benchmarks/benchmark_sampling.py:21-23  (mask y < k-th largest);
 *   - top-p on the descending order: benchmarks/benchmark_sampling.py:25-34
 *     (softmax of the sorted row, cumulative sum, remove where the sum before an entry
 *     exceeds p, the first entry always stays);
 *   - final softmax + one draw: benchmarks/benchmark_sampling.py:36-37.
 * Two things the reference leaves to torch internals are fixed by convention here:
 * equal values are ordered by ascending vocabulary index (the reference's sort is
 * unstable), and the draw is an inverse CDF over the survivors in ascending index
 * order driven by one caller-supplied uniform (the reference's multinomial consumes
 * torch's RNG stream).
 *
 * Arithmetic is specified so that any machine reproduces it bit for bit: softmax
 * masses are W(y - max) = trunc(2^40 * exp(y - max)) with exp evaluated by the fixed
 * sequence of IEEE-754 double operations in ka_oracle_weight(), masses are summed as
 * 64-bit integers (order-free), and both thresholds (top_p * Z and u * Z) are exact
 * integer floors of the fp32 scalar times the integer total.  Compile with
 * -ffp-contract=off.
 *
 * Pinned by tests/test_oracle_sampling.py: a pure-Python big-rational evaluation of
 * the same definition on small rows, the torch restatement (oracle/sampling_ref.py) on
 * seeded rows, and closed forms (top_k=1 is argmax for every u; u=0 gives the
 * smallest surviving index; u->1 the largest; top_p->0 keeps the argmax; uniform rows
 * keep ceil-counts; stratified uniforms reproduce the probabilities).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define KA_DTYPE_BF16 0
#define KA_DTYPE_F16 1
#define KA_DTYPE_F32 2

#define KA_FIX_BITS 40

typedef unsigned __int128 u128;

static float bits_to_f32(uint32_t b) { float f; memcpy(&f, &b, 4); return f; }
static uint32_t f32_to_bits(float f) { uint32_t b; memcpy(&b, &f, 4); return b; }

/* ---- dtype conversions (round to nearest even) ------------------------------------ */
static float bf16_to_f32(uint16_t h) { return bits_to_f32((uint32_t)h << 16); }
static uint16_t f32_to_bf16(float f) {
    uint32_t b = f32_to_bits(f);
    if ((b & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((b >> 16) | 0x40); /* NaN */
    b += 0x7fffu + ((b >> 16) & 1u);
    return (uint16_t)(b >> 16);
}
static float f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu, man = h & 0x3ffu;
    if (exp == 0) {
        if (man == 0) return bits_to_f32(sign);
        float v = (float)man * (1.0f / 16777216.0f); /* man * 2^-24, exact */
        return sign ? -v : v;
    }
    if (exp == 31) return bits_to_f32(sign | 0x7f800000u | (man << 13));
    return bits_to_f32(sign | ((exp + 112u) << 23) | (man << 13));
}
static uint16_t f32_to_f16(float f) {
    uint32_t b = f32_to_bits(f);
    uint16_t sign = (uint16_t)((b >> 16) & 0x8000u);
    uint32_t a = b & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);          /* NaN */
    if (a >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);         /* >= 65520 rounds to inf */
    if (a < 0x33000001u) return sign;                                /* <= 2^-25 rounds to 0 */
    if (a < 0x38800000u) {                                           /* subnormal half */
        /* value = a_float; result mantissa = round(value * 2^24) */
        uint32_t e = a >> 23, m = (a & 0x7fffffu) | 0x800000u;
        uint32_t shift = 126u - e;                                   /* 14..24 */
        uint32_t q = m >> shift, rem = m & ((1u << shift) - 1u), half = 1u << (shift - 1);
        if (rem > half || (rem == half && (q & 1u))) q++;
        return (uint16_t)(sign | q);
    }
    uint32_t q = (a - 0x38000000u) >> 13, rem = a & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) q++;
    return (uint16_t)(sign | q);
}

/* y = x / T in the row's dtype; -0 is folded into +0 so that equal values have equal keys. */
static float load_scaled(const void *row, int dtype, int64_t i, float T) {
    float x, y;
    switch (dtype) {
        case KA_DTYPE_BF16:
            x = bf16_to_f32(((const uint16_t *)row)[i]);
            y = (T != 1.0f) ? bf16_to_f32(f32_to_bf16(x / T)) : x;
            break;
        case KA_DTYPE_F16:
            x = f16_to_f32(((const uint16_t *)row)[i]);
            y = (T != 1.0f) ? f16_to_f32(f32_to_f16(x / T)) : x;
            break;
        default:
            x = ((const float *)row)[i];
            y = (T != 1.0f) ? x / T : x;
            break;
    }
    if (y == 0.0f) y = 0.0f;
    return y;
}

/* Order-preserving map fp32 -> uint32 (larger float <=> larger key). */
static uint32_t key_of(float y) {
    uint32_t b = f32_to_bits(y);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

/*
 * W(d) = trunc(2^40 * exp(d)) for d <= 0, by a fixed sequence of IEEE double operations:
 *   t = d * log2(e);  n = trunc(t - 0.5);  f = t - n  (|f| <= 0.5);  g = f * ln 2;
 *   p = sum_{k=0..11} g^k / k!  (Horner with fma(), one rounding per step);  W = trunc(p * 2^(40+n)).
 * W(0) = 2^40 exactly; W(d) = 0 once t < -41.
 */
/* One body, compiled twice: with the hardware fused multiply-add where the CPU has one, and with libm's
 * fma() (exact by C99) elsewhere.  Both round each Horner step once, so they return the same integers. */
#define KA_WEIGHT_BODY(FMA)                                                                               \
    static const double C[12] = {0x1.0000000000000p+0,  0x1.0000000000000p+0,  0x1.0000000000000p-1,      \
                                 0x1.5555555555555p-3,  0x1.5555555555555p-5,  0x1.1111111111111p-7,      \
                                 0x1.6c16c16c16c17p-10, 0x1.a01a01a01a01ap-13, 0x1.a01a01a01a01ap-16,     \
                                 0x1.71de3a556c734p-19, 0x1.27e4fb7789f5cp-22, 0x1.ae64567f544e4p-26};    \
    const double LOG2E = 0x1.71547652b82fep+0, LN2 = 0x1.62e42fefa39efp-1;                                \
    if (!(d <= 0.0f)) return d > 0.0f ? (uint64_t)1 << KA_FIX_BITS : 0; /* d > 0 cannot occur; NaN -> 0 */ \
    double t = (double)d * LOG2E;                                                                         \
    if (t < -41.0) return 0;                                                                              \
    int n = (int)(t - 0.5);                                                                               \
    double f = t - (double)n;                                                                             \
    double g = f * LN2;                                                                                   \
    double p = C[11];                                                                                     \
    for (int k = 10; k >= 0; --k) p = FMA(p, g, C[k]);                                                    \
    uint64_t pow2_bits = (uint64_t)(1023 + KA_FIX_BITS + n) << 52;                                        \
    double scale;                                                                                         \
    memcpy(&scale, &pow2_bits, 8);                                                                        \
    return (uint64_t)(p * scale);

__attribute__((target("fma"))) static uint64_t weight_hw(float d) { KA_WEIGHT_BODY(__builtin_fma) }
static uint64_t weight_sw(float d) { KA_WEIGHT_BODY(fma) }

uint64_t ka_oracle_weight(float d) {
    static int have_fma = -1;
    if (have_fma < 0) have_fma = __builtin_cpu_supports("fma") ? 1 : 0;
    return have_fma ? weight_hw(d) : weight_sw(d);
}

/* The libm-fma() build of the same function, exported for the test that compares the two. */
uint64_t ka_oracle_weight_libm(float d) { return weight_sw(d); }

/* floor(s * z) for an fp32 scalar 0 <= s < 1 and an integer z < 2^62, exactly. */
static uint64_t floor_scale(float s, uint64_t z) {
    uint32_t b = f32_to_bits(s);
    uint32_t e = (b >> 23) & 0xffu, m = b & 0x7fffffu;
    if (e == 0 && m == 0) return 0;
    int shift; /* s = mant * 2^-shift */
    uint64_t mant;
    if (e == 0) { mant = m; shift = 149; } else { mant = m | 0x800000u; shift = 150 - (int)e; }
    u128 prod = (u128)mant * (u128)z;
    if (shift >= 128) return 0;
    return (uint64_t)(prod >> shift);
}

typedef struct { uint32_t key; int32_t idx; } cand_t;

static int cmp_key_desc_idx_asc(const void *a, const void *b) {
    const cand_t *x = (const cand_t *)a, *y = (const cand_t *)b;
    if (x->key != y->key) return x->key > y->key ? -1 : 1;
    return x->idx < y->idx ? -1 : (x->idx > y->idx ? 1 : 0);
}
static int cmp_idx_asc(const void *a, const void *b) {
    const cand_t *x = (const cand_t *)a, *y = (const cand_t *)b;
    return x->idx < y->idx ? -1 : (x->idx > y->idx ? 1 : 0);
}

/* k-th largest key (1 <= k <= n) by two 16-bit counting passes. */
static uint32_t kth_largest_key(const uint32_t *keys, int64_t n, int64_t k, int64_t *hist) {
    memset(hist, 0, 65536 * sizeof(int64_t));
    for (int64_t i = 0; i < n; ++i) hist[keys[i] >> 16]++;
    int64_t above = 0;
    int hi = 65535;
    for (; hi >= 0; --hi) {
        if (above + hist[hi] >= k) break;
        above += hist[hi];
    }
    memset(hist, 0, 65536 * sizeof(int64_t));
    for (int64_t i = 0; i < n; ++i)
        if ((int)(keys[i] >> 16) == hi) hist[keys[i] & 0xffffu]++;
    int lo = 65535;
    for (; lo >= 0; --lo) {
        if (above + hist[lo] >= k) break;
        above += hist[lo];
    }
    return ((uint32_t)hi << 16) | (uint32_t)lo;
}

/* Per-row diagnostics (all optional outputs of ka_oracle_sample). */
typedef struct {
    int64_t n_topk;   /* |A|: entries surviving top-k (ties included) */
    int64_t n_kept;   /* |B|: entries surviving top-p */
    uint64_t z_topk;  /* integer mass of A */
    uint64_t z_kept;  /* integer mass of B */
    float kth_value;  /* k-th largest scaled logit (or -inf when top-k is off) */
    float max_value;
    uint64_t w_pick;  /* integer mass of the sampled entry: its probability is w_pick / z_kept */
} ka_oracle_row_info;

int ka_oracle_sample(const void *logits, int dtype, int64_t batch, int64_t vocab, int64_t row_stride,
                     float temperature, int32_t top_k, float top_p, const float *uniforms,
                     int64_t *out_ids, ka_oracle_row_info *info) {
    if (batch < 0 || vocab < 1 || vocab >= ((int64_t)1 << 22) || row_stride < vocab) return -1;
    if (!(temperature > 0.0f) || top_k < 0 || !(top_p > 0.0f && top_p <= 1.0f)) return -1;
    if (dtype != KA_DTYPE_BF16 && dtype != KA_DTYPE_F16 && dtype != KA_DTYPE_F32) return -1;
    const size_t esize = dtype == KA_DTYPE_F32 ? 4 : 2;
    float *y = (float *)malloc((size_t)vocab * sizeof(float));
    uint32_t *keys = (uint32_t *)malloc((size_t)vocab * sizeof(uint32_t));
    cand_t *cand = (cand_t *)malloc((size_t)vocab * sizeof(cand_t));
    uint64_t *w = (uint64_t *)malloc((size_t)vocab * sizeof(uint64_t));
    int64_t *hist = (int64_t *)malloc(65536 * sizeof(int64_t));
    if (!y || !keys || !cand || !w || !hist) { free(y); free(keys); free(cand); free(w); free(hist); return -2; }

    for (int64_t r = 0; r < batch; ++r) {
        const void *row = (const char *)logits + (size_t)r * (size_t)row_stride * esize;
        /* 1. temperature; 2. keys */
        float mx = -INFINITY;
        for (int64_t i = 0; i < vocab; ++i) {
            y[i] = load_scaled(row, dtype, i, temperature);
            if (y[i] != y[i]) y[i] = -INFINITY; /* a NaN logit counts as -inf (the reference would fail on it) */
            keys[i] = key_of(y[i]);
            if (i == 0 || keys[i] > key_of(mx)) mx = y[i];
        }
        /* 3. top-k threshold, ties kept */
        uint32_t kth = 0;
        if (top_k > 0 && (int64_t)top_k < vocab) kth = kth_largest_key(keys, vocab, top_k, hist);
        int64_t na = 0;
        for (int64_t i = 0; i < vocab; ++i)
            if (keys[i] >= kth) { cand[na].key = keys[i]; cand[na].idx = (int32_t)i; na++; }
        /* 4. integer masses relative to the row maximum */
        qsort(cand, (size_t)na, sizeof(cand_t), cmp_key_desc_idx_asc);
        uint64_t za = 0;
        for (int64_t j = 0; j < na; ++j) {
            float v = y[cand[j].idx];
            float d = (v == mx) ? 0.0f : v - mx;
            w[j] = ka_oracle_weight(d);
            za += w[j];
        }
        /* 5. top-p: keep position j iff the mass strictly before it is <= top_p * Z */
        int64_t nb = na;
        if (top_p < 1.0f) {
            uint64_t theta = floor_scale(top_p, za);
            uint64_t before = 0;
            nb = 0;
            for (int64_t j = 0; j < na; ++j) {
                if (before > theta) break;
                nb++;
                before += w[j];
            }
        }
        uint64_t zb = 0;
        for (int64_t j = 0; j < nb; ++j) zb += w[j];
        /* 6. inverse CDF over the survivors in ascending index order */
        for (int64_t j = 0; j < nb; ++j) cand[j].key = (uint32_t)j; /* remember the mass slot */
        qsort(cand, (size_t)nb, sizeof(cand_t), cmp_idx_asc);
        float u = uniforms[r];
        if (!(u >= 0.0f)) u = 0.0f;
        if (u >= 1.0f) u = bits_to_f32(0x3f7fffffu);
        uint64_t tau = floor_scale(u, zb);
        uint64_t cum = 0;
        int64_t pick = cand[nb - 1].idx;
        uint64_t w_pick = w[cand[nb - 1].key];
        for (int64_t j = 0; j < nb; ++j) {
            cum += w[cand[j].key];
            if (cum > tau) { pick = cand[j].idx; w_pick = w[cand[j].key]; break; }
        }
        out_ids[r] = pick;
        if (info) {
            info[r].n_topk = na;
            info[r].n_kept = nb;
            info[r].z_topk = za;
            info[r].z_kept = zb;
            info[r].kth_value = kth ? bits_to_f32((kth & 0x80000000u) ? (kth & 0x7fffffffu) : ~kth) : -INFINITY;
            info[r].max_value = mx;
            info[r].w_pick = w_pick;
        }
    }
    free(y); free(keys); free(cand); free(w); free(hist);
    return 0;
}

/* Element-wise helpers exported for the tests. */
void ka_oracle_scale(const void *src, int dtype, int64_t n, float temperature, float *dst) {
    for (int64_t i = 0; i < n; ++i) dst[i] = load_scaled(src, dtype, i, temperature);
}
uint64_t ka_oracle_floor_scale(float s, uint64_t z) { return floor_scale(s, z); }

/*
 * oracle_kernels.c — bit-level CPU checkers for the dispatch/combine hot path.
 *
 * TEST INFRASTRUCTURE ONLY: loaded by tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py.  The product library never links or calls it.
 *
 * What is here is written independently of the torch oracle so that the two
 * pin each other:
 *   - an OCP e4m3fn encoder from the format definition (1-4-3, bias 7, no
 *     infinities, 0x7f = NaN, round to nearest even), against torch's cast;
 *   - the per-token cast of csrc/kernels/efa_kernels.cu:143-169 in scalar C;
 *   - the combine accumulation of csrc/kernels/coop_combine_recv.cuh:247-256
 *     with a true fmaf per step;
 *   - the integer hashes of the seeded loopback world.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

static inline float bits_to_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f32_to_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bf16_to_f32(uint16_t b) { return bits_to_f32((uint32_t)b << 16); }

static inline uint16_t f32_to_bf16(float f) {
    uint32_t u = f32_to_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

/* float32 -> e4m3fn byte.  Values that round above 448 give NaN (0x7f), as an
 * unsaturated conversion does; callers clamp first. */
uint8_t oracle_e4m3_encode(float f) {
    const uint32_t u = f32_to_bits(f);
    const uint8_t sign = (uint8_t)((u >> 31) << 7);
    const uint32_t au = u & 0x7fffffffu;
    if (au > 0x7f800000u) return sign | 0x7f;
    const float a = bits_to_f32(au);
    if (a < 0.015625f) { /* below 2^-6: subnormal grid of 2^-9 */
        const float q = nearbyintf(a * 512.0f); /* exact scaling, ties to even */
        return sign | (uint8_t)q;               /* q == 8 is the smallest normal, 0x08 */
    }
    int exp = (int)(au >> 23) - 127;
    uint32_t mant = au & 0x7fffffu;
    uint32_t m3 = mant >> 20;
    const uint32_t rest = mant & 0xfffffu;
    if (rest > 0x80000u || (rest == 0x80000u && (m3 & 1u))) m3 += 1;
    if (m3 == 8) { m3 = 0; exp += 1; }
    if (exp > 8 || (exp == 8 && m3 == 7)) return sign | 0x7f;
    return sign | (uint8_t)(((exp + 7) << 3) | m3);
}

float oracle_e4m3_decode(uint8_t b) {
    const int sign = b >> 7, ex = (b >> 3) & 15, m = b & 7;
    float v;
    if (ex == 15 && m == 7) return NAN;
    if (ex == 0) v = ldexpf((float)m, -9);
    else v = ldexpf(1.0f + (float)m / 8.0f, ex - 7);
    return sign ? -v : v;
}

void oracle_e4m3_encode_many(const float* in, uint8_t* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = oracle_e4m3_encode(in[i]);
}

static inline float clamp448(float v) { return fminf(fmaxf(v, -448.0f), 448.0f); }

/* fmt: 1 = float32 scales amax/448, 2 = power-of-two float32 scales,
 * 3 = power-of-two scales stored as exponent bytes.
 * x [rows, cols] bf16 bits; q [rows, cols]; scales: 4 bytes per group (fmt 1, 2)
 * or 1 byte per group (fmt 3). */
void oracle_per_token_cast(const uint16_t* x, int64_t rows, int cols, int fmt, uint8_t* q, uint8_t* scales) {
    const int groups = cols / 128;
    for (int64_t r = 0; r < rows; ++r) {
        for (int g = 0; g < groups; ++g) {
            const uint16_t* src = x + r * cols + (int64_t)g * 128;
            float amax = 0.0f;
            for (int i = 0; i < 128; ++i) amax = fmaxf(amax, fabsf(bf16_to_f32(src[i])));
            amax = fmaxf(amax, 1e-4f);
            float scale = amax / 448.0f, inv = 448.0f / amax;
            if (fmt != 1) {
                uint32_t bits = f32_to_bits(scale);
                uint32_t ex = (bits >> 23) & 0xffu;
                if (bits & 0x7fffffu) ex += 1;
                scale = bits_to_f32(ex << 23);
                inv = 1.0f / scale;
            }
            for (int i = 0; i < 128; ++i)
                q[r * cols + (int64_t)g * 128 + i] = oracle_e4m3_encode(clamp448(bf16_to_f32(src[i]) * inv));
            if (fmt == 3) {
                scales[r * groups + g] = (uint8_t)(f32_to_bits(scale) >> 23);
            } else {
                const uint32_t sb = f32_to_bits(scale);
                memcpy(scales + (r * groups + g) * 4, &sb, 4);
            }
        }
    }
}

/* out[t,h] = bf16( chain over k of fmaf(f32(rows[t,k,h]), w[t,k], acc) ), skipping dead pairs. */
void oracle_combine_chain(const uint16_t* rows, const float* weights, const uint8_t* live, int64_t tokens,
                          int topk, int hidden, uint16_t* out) {
    for (int64_t t = 0; t < tokens; ++t)
        for (int h = 0; h < hidden; ++h) {
            float acc = 0.0f;
            for (int k = 0; k < topk; ++k) {
                if (!live[t * topk + k]) continue;
                acc = fmaf(bf16_to_f32(rows[(t * topk + k) * (int64_t)hidden + h]), weights[t * topk + k], acc);
            }
            out[t * hidden + h] = f32_to_bf16(acc);
        }
}

/* ---- seeded world ---------------------------------------------------- */
static inline uint32_t mix32(uint32_t x) {
    x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
    return x;
}
static inline uint32_t row_hash(uint32_t seed, uint32_t key) { return mix32(seed ^ mix32(key + 0x9e3779b9u)); }

uint32_t oracle_mix32(uint32_t x) { return mix32(x); }

void oracle_synth_bf16_rows(const uint32_t* keys, int64_t num_rows, int hidden, uint32_t seed, int outlier_period,
                            uint16_t* out) {
    const float unit = bits_to_f32(0x3bddb47bu);
    for (int64_t r = 0; r < num_rows; ++r) {
        const uint32_t rh = row_hash(seed, keys[r]);
        const int hot = outlier_period > 0 && (mix32(rh ^ 0x5bd1e995u) % (uint32_t)outlier_period) == 0;
        for (int c = 0; c < hidden; ++c) {
            const uint32_t h = mix32(rh ^ ((uint32_t)c * 0x9e3779b1u + 0x85ebca6bu));
            const int s = (int)(h & 255u) + (int)((h >> 8) & 255u) + (int)((h >> 16) & 255u) + (int)(h >> 24);
            float f = (float)(s - 510) * unit;
            if (hot) f = f * 100.0f;
            out[r * hidden + c] = f32_to_bf16(f);
        }
    }
}

void oracle_synth_topk_idx(const uint32_t* cdf, const int32_t* ranks, int num_src, int num_tokens, int num_topk,
                           int num_experts, uint32_t seed, int64_t* out) {
    for (int b = 0; b < num_src; ++b)
        for (int t = 0; t < num_tokens; ++t) {
            const uint32_t th = row_hash(seed ^ 0x7f4a7c15u, (uint32_t)ranks[b] * (uint32_t)num_tokens + (uint32_t)t);
            int64_t* row = out + ((int64_t)b * num_tokens + t) * num_topk;
            int have = 0;
            for (int c = 0; c < 64 * num_topk && have < num_topk; ++c) {
                const uint32_t u = mix32(th + (uint32_t)c * 0x9e3779b9u);
                int lo = 0, hi = num_experts - 1;
                while (lo < hi) {
                    const int mid = (lo + hi) >> 1;
                    if (cdf[mid] >= u) hi = mid; else lo = mid + 1;
                }
                int seen = 0;
                for (int j = 0; j < have; ++j) seen |= row[j] == lo;
                if (!seen) row[have++] = lo;
            }
            for (int e = 0; e < num_experts && have < num_topk; ++e) {
                int seen = 0;
                for (int j = 0; j < have; ++j) seen |= row[j] == e;
                if (!seen) row[have++] = e;
            }
        }
}

/* CPU oracle for the decode+matmul path, plain C.  TEST INFRASTRUCTURE ONLY.
 *
 * A second, independent restatement (scalar loops, software IEEE half) of what
 * oracle/dmm_oracle.py states with numpy; the tests require the two to agree bit for
 * bit, and the HIP kernels are checked against them.  Nothing shipped links this file.
 *
 * Reference lines followed:
 *   code fields, flip-then-shift decode ... /root/reference/test_decode_matmul.py:29-55
 *   SWAR decoder .......................... /root/reference/decode_matmul_cuda/decode_matmul_cuda.cu:45-65
 *   W[n, 8*j+d] index convention, matmul .. /root/reference/test_decode_matmul.py:58-71
 */
#include <stdint.h>
#include <string.h>

/* ---- software IEEE binary16 <-> binary32 -------------------------------------- */
static float half_to_float(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {                       /* subnormal: normalise */
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            man &= 0x3FFu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* round-to-nearest-even float -> half */
static uint16_t float_to_half(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t absx = x & 0x7FFFFFFFu;
    if (absx >= 0x7F800000u) {                      /* inf / nan */
        uint32_t man = absx & 0x7FFFFFu;
        return (uint16_t)(sign | 0x7C00u | (man ? (0x200u | (man >> 13)) : 0));
    }
    if (absx >= 0x477FF000u)                        /* >= 65520 rounds to inf */
        return (uint16_t)(sign | 0x7C00u);
    if (absx < 0x33000001u)                         /* <= 2^-25 rounds to zero (tie -> even = 0) */
        return (uint16_t)sign;
    int32_t e = (int32_t)(absx >> 23) - 127;
    uint32_t man = (absx & 0x7FFFFFu) | 0x800000u;  /* 24-bit significand */
    int shift;                                      /* bits to drop */
    uint32_t base;
    if (e < -14) {                                  /* subnormal half */
        shift = 13 + (-14 - e);
        base = 0;
    } else {
        shift = 13;
        base = (uint32_t)(e + 15) << 10;
        man &= 0x7FFFFFu;
    }
    uint32_t kept = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1);
    uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (kept & 1)))
        kept++;                                     /* carry may ripple into the exponent: correct */
    return (uint16_t)(sign | (base + kept));
}

/* ---- code fields (test_decode_matmul.py:30-33) -------------------------------- */
static inline unsigned sign8(uint16_t c)
{
    unsigned s7 = (c >> 8) & 0x7Fu;
    unsigned p = 0;
    for (int i = 0; i < 7; i++) p ^= (s7 >> i) & 1u;
    return s7 | (p << 7);
}

/* fp16 decode of n_codes codes; W receives 8 halves per code. */
void dmm_oracle_decode_f16(const uint16_t *codes, const uint16_t *grid,
                           uint16_t *W, int64_t n_codes)
{
    for (int64_t i = 0; i < n_codes; i++) {
        uint16_t c = codes[i];
        unsigned idx = c & 0xFFu;
        unsigned s8 = sign8(c);
        float delta = (c >> 15) ? -0.25f : 0.25f;
        for (int d = 0; d < 8; d++) {
            uint16_t g = grid[idx * 8 + d];
            if ((s8 >> d) & 1u) g ^= 0x8000u;             /* flip first ... */
            /* ... then add: the fp32 sum of a half and +-0.25 is exact, so a single
             * rounding to half equals the IEEE half add. */
            W[i * 8 + d] = float_to_half(half_to_float(g) + delta);
        }
    }
}

/* literal int8 decode (test_decode_matmul.py:35-52) */
void dmm_oracle_decode_i8(const uint16_t *codes, const int64_t *codebook_abs,
                          int8_t *W, int64_t n_codes)
{
    for (int64_t i = 0; i < n_codes; i++) {
        uint16_t c = codes[i];
        uint64_t abs = (uint64_t)codebook_abs[c & 0xFFu];
        unsigned s8 = sign8(c);
        int shift = (c >> 15) & 1;
        for (int d = 0; d < 8; d++) {
            int8_t v = (int8_t)(abs & 0xFFu);
            if (s8 & 1u) v = (int8_t)(-v);
            v = (int8_t)(shift ? v - 1 : v + 1);
            W[i * 8 + d] = v;
            abs >>= 8;
            s8 >>= 1;
        }
    }
}

/* the CUDA kernel's SWAR decoder (decode_matmul_cuda.cu:45-65), one uint64 per code */
void dmm_oracle_decode_swar(const uint16_t *codes, const int64_t *codebook_abs,
                            uint64_t *out, int64_t n_codes)
{
    for (int64_t i = 0; i < n_codes; i++) {
        uint16_t c = codes[i];
        uint8_t bits_abs = c & 0xFF;
        uint8_t bits_sign = (c >> 8) & 0x7F;
        uint64_t bit_shift = (c >> 15) & 1;
        uint64_t s = bits_sign | ((uint64_t)(__builtin_popcount(bits_sign) & 1) << 7);
        s |= s << 28;
        s |= s << 14;
        s |= s << 7;
        s &= 0x0101010101010101ull;
        s *= 252;
        uint64_t packed = (uint64_t)codebook_abs[bits_abs] ^ s;
        packed -= bit_shift * 0x0202020202020202ull;
        packed |= 0x0101010101010101ull;
        out[i] = packed;
    }
}

/* y[m,n] = scale * sum_k x[m,k] * W[n,k]; halves in, float out, double accumulate */
void dmm_oracle_matmul_f16(const uint16_t *x, const uint16_t *W, float scale,
                           float *y, int64_t M, int64_t N, int64_t K)
{
    for (int64_t m = 0; m < M; m++)
        for (int64_t n = 0; n < N; n++) {
            double acc = 0.0;
            for (int64_t k = 0; k < K; k++)
                acc += (double)half_to_float(x[m * K + k]) * (double)half_to_float(W[n * K + k]);
            y[m * N + n] = (float)(acc * (double)scale);
        }
}

/* integer operator (test_decode_matmul.py:58-71): codes un-tiled [N, K/8] */
void dmm_oracle_decode_matmul_i32(const int8_t *x, const uint16_t *codes,
                                  const int64_t *codebook_abs, int32_t *out,
                                  int64_t M, int64_t N, int64_t K)
{
    int8_t w[8];
    for (int64_t m = 0; m < M; m++)
        for (int64_t n = 0; n < N; n++) {
            int32_t acc = 0;
            for (int64_t j = 0; j < K / 8; j++) {
                dmm_oracle_decode_i8(&codes[n * (K / 8) + j], codebook_abs, w, 1);
                for (int d = 0; d < 8; d++)
                    acc += (int32_t)x[m * K + 8 * j + d] * (int32_t)w[d];
            }
            out[m * N + n] = acc;
        }
}

/* exposed for the half-conversion tests */
uint16_t dmm_oracle_f2h(float f) { return float_to_half(f); }
float dmm_oracle_h2f(uint16_t h) { return half_to_float(h); }

/* Stand-alone driver for the C oracle, built with -fsanitize=address,undefined.
 * Runs every entry point over all 65536 codes and a small matmul so that an
 * out-of-bounds access or undefined shift in the oracle itself is caught on the host.
 * TEST INFRASTRUCTURE ONLY. */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

void dmm_oracle_decode_f16(const uint16_t *, const uint16_t *, uint16_t *, int64_t);
void dmm_oracle_decode_i8(const uint16_t *, const int64_t *, int8_t *, int64_t);
void dmm_oracle_decode_swar(const uint16_t *, const int64_t *, uint64_t *, int64_t);
void dmm_oracle_matmul_f16(const uint16_t *, const uint16_t *, float, float *, int64_t, int64_t, int64_t);
void dmm_oracle_decode_matmul_i32(const int8_t *, const uint16_t *, const int64_t *, int32_t *, int64_t, int64_t, int64_t);
uint16_t dmm_oracle_f2h(float);
float dmm_oracle_h2f(uint16_t);

int main(void)
{
    enum { NC = 65536 };
    uint16_t *codes = malloc(NC * 2), *grid = malloc(256 * 8 * 2), *W = malloc((size_t)NC * 16);
    int64_t *cb = malloc(256 * 8);
    int8_t *Wi = malloc((size_t)NC * 8);
    uint64_t *sw = malloc((size_t)NC * 8);
    for (int i = 0; i < NC; i++) codes[i] = (uint16_t)i;
    for (int i = 0; i < 256; i++) {
        uint64_t p = 0;
        for (int d = 0; d < 8; d++) {
            int q = 2 + 4 * ((i * 7 + d * 3) % 3);            /* 2, 6, 10 */
            if (d == 7 && (i & 1)) q = 256 - q;
            p |= (uint64_t)q << (8 * d);
            grid[i * 8 + d] = dmm_oracle_f2h((float)(int8_t)q / 4.0f);
        }
        cb[i] = (int64_t)p;
    }
    dmm_oracle_decode_f16(codes, grid, W, NC);
    dmm_oracle_decode_i8(codes, cb, Wi, NC);
    dmm_oracle_decode_swar(codes, cb, sw, NC);
    long bad = 0;
    for (long i = 0; i < (long)NC * 8; i++) {
        if (dmm_oracle_h2f(W[i]) * 4.0f != (float)Wi[i]) bad++;
        if ((int8_t)((sw[i / 8] >> (8 * (i % 8))) & 0xFF) != Wi[i]) bad++;
    }
    /* every half survives a round trip through float */
    for (uint32_t h = 0; h < 65536; h++) {
        uint16_t e = (uint16_t)h;
        if ((e & 0x7C00) == 0x7C00 && (e & 0x3FF)) continue;  /* NaN payloads aside */
        if (dmm_oracle_f2h(dmm_oracle_h2f(e)) != e) bad++;
    }
    enum { M = 3, N = 5, K = 64 };
    uint16_t x[M * K];
    int8_t xi[M * K];
    float y[M * N];
    int32_t yi[M * N];
    for (int i = 0; i < M * K; i++) { xi[i] = (int8_t)(i * 37 - 90); x[i] = dmm_oracle_f2h((float)xi[i]); }
    dmm_oracle_matmul_f16(x, W, 1.0f, y, M, N, K);
    dmm_oracle_decode_matmul_i32(xi, codes, cb, yi, M, N, K);
    for (int i = 0; i < M * N; i++)
        if (y[i] * 4.0f != (float)yi[i]) bad++;
    printf("oracle_selftest mismatches=%ld\n", bad);
    free(codes); free(grid); free(W); free(cb); free(Wi); free(sw);
    return bad != 0;
}

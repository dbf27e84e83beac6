/* Runs every oracle function on small ragged inputs; built with -fsanitize=address,undefined
 * by tests/test_host_cpu.py so that out-of-bounds accesses in the oracle itself show up. */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

int lpmm_oracle_qmapping(const float *qmap, int bits, float x);
void lpmm_oracle_pack_nonlinear_4bit(const float *x, const float *qmap, int64_t n_padded, uint8_t *out);
void lpmm_oracle_unpack_nonlinear_4bit(const uint8_t *codes, const float *qmap, int64_t n, float *out);
void lpmm_oracle_adamw_fp32_step(float *p, const float *g, float *m, float *v, int64_t n, float, float, float, float, float, float);
void lpmm_oracle_adamw4bit_step(float *p, const float *g, uint8_t *mc, uint8_t *vc, float *ms, float *vs, const float *qm,
                                const float *qv, int64_t n, float, float, float, float, float, float);
void lpmm_oracle_quant_group(const float *x, int64_t n, int64_t gp, const float *qmap, uint8_t *codes, float *max1);
void lpmm_oracle_dequant_group(const uint8_t *codes, const float *max1, const float *qmap, int64_t n, int64_t gp, float *out);
void lpmm_oracle_rank1_stats(const float *x, int64_t R, int64_t C, float *rowmax, float *colmax);
void lpmm_oracle_quant_rank1(const float *x, int64_t R, int64_t C, const float *rowmax, const float *colmax, const float *qmap, uint8_t *codes);
void lpmm_oracle_dequant_rank1(const uint8_t *codes, const float *rowmax, const float *colmax, const float *qmap, int64_t R, int64_t C, float *out);
void lpmm_oracle_nonfused_update(float *p, const float *g, float *m, float *v, int64_t n, double, double, double, double, double, double);
void lpmm_oracle_factored_stats(const float *g, int64_t R, int64_t C, float *row_mean, float *col_mean);
float lpmm_oracle_factored_ema(float *row, float *col, const float *row_mean, const float *col_mean, int64_t R, int64_t C, double beta2);
void lpmm_oracle_factored_update(float *p, const float *g, float *m, const float *row, const float *col, float mean_all,
                                 int64_t R, int64_t C, double, double, double, double, double, double);

static float *fl(int64_t n, float scale) {
    float *a = malloc(sizeof(float) * (size_t)(n > 0 ? n : 1));
    for (int64_t i = 0; i < n; ++i) a[i] = scale * (float)((i * 2654435761u) % 1000 - 500) / 500.0f;
    return a;
}

int main(void) {
    float qm[16], qv[16];
    for (int k = 0; k < 16; ++k) { qv[k] = (k + 1) / 16.0f; qm[k] = (k - 7) / 8.0f; }
    if (lpmm_oracle_qmapping(qm, 4, NAN) != -1) return 2;
    const int64_t sizes[] = {1, 2, 7, 127, 128, 129, 2047, 2049, 4097};
    for (size_t s = 0; s < sizeof sizes / sizeof *sizes; ++s) {
        const int64_t n = sizes[s], nb = (n + 1) / 2, ng = (n + 127) / 128;
        float *p = fl(n, 0.02f), *g = fl(n, 1e-3f), *m = calloc((size_t)n, 4), *v = calloc((size_t)n, 4);
        uint8_t *mc = calloc((size_t)nb, 1), *vc = calloc((size_t)nb, 1);
        float *ms = calloc((size_t)ng, 4), *vs = calloc((size_t)ng, 4);
        for (int step = 1; step <= 2; ++step) {
            lpmm_oracle_adamw4bit_step(p, g, mc, vc, ms, vs, qm, qv, n, 0.9f, 0.999f, 1e-3f, 0.01f, 1e-8f, (float)step);
            lpmm_oracle_adamw_fp32_step(p, g, m, v, n, 0.9f, 0.999f, 1e-3f, 0.01f, 1e-8f, (float)step);
            lpmm_oracle_nonfused_update(p, g, m, v, n, 0.9, 0.999, 1e-3, 0.01, 1e-8, (double)step);
        }
        for (int64_t gp = 128; gp <= 2048; gp *= 4) {
            const int64_t G = (n + gp - 1) / gp, NG = (G * gp + 2047) / 2048;
            uint8_t *codes = malloc((size_t)(NG * 1024 + 1));
            float *max1 = malloc(sizeof(float) * (size_t)G), *out = malloc(sizeof(float) * (size_t)n);
            lpmm_oracle_quant_group(g, n, gp, qm, codes, max1);
            lpmm_oracle_dequant_group(codes, max1, qm, n, gp, out);
            float *un = malloc(sizeof(float) * (size_t)(NG * 2048));
            lpmm_oracle_unpack_nonlinear_4bit(codes, qm, NG * 2048, un);
            free(un);
            free(codes); free(max1); free(out);
        }
        free(p); free(g); free(m); free(v); free(mc); free(vc); free(ms); free(vs);
    }
    const int64_t shapes[][2] = {{1, 1}, {3, 5}, {64, 33}, {17, 300}};
    for (size_t s = 0; s < 4; ++s) {
        const int64_t R = shapes[s][0], C = shapes[s][1], n = R * C, NG = (n + 2047) / 2048;
        float *x = fl(n, 1.0f), *p = fl(n, 0.02f), *m = calloc((size_t)n, 4), *out = malloc(sizeof(float) * (size_t)n);
        float *row = calloc((size_t)R, 4), *col = calloc((size_t)C, 4), *rm = malloc(sizeof(float) * (size_t)R), *cm = malloc(sizeof(float) * (size_t)C);
        uint8_t *codes = malloc((size_t)(NG * 1024 + 1));
        lpmm_oracle_rank1_stats(x, R, C, rm, cm);
        lpmm_oracle_quant_rank1(x, R, C, rm, cm, qv, codes);
        lpmm_oracle_dequant_rank1(codes, rm, cm, qv, R, C, out);
        lpmm_oracle_factored_stats(x, R, C, rm, cm);
        const float mean_all = lpmm_oracle_factored_ema(row, col, rm, cm, R, C, 0.999);
        lpmm_oracle_factored_update(p, x, m, row, col, mean_all, R, C, 0.9, 0.999, 1e-3, 0.01, 1e-8, 1.0);
        float *pk = fl(NG * 2048, 1.0f);
        lpmm_oracle_pack_nonlinear_4bit(pk, qm, NG * 2048, codes);
        free(pk); free(x); free(p); free(m); free(out); free(row); free(col); free(rm); free(cm); free(codes);
    }
    puts("ok");
    return 0;
}

/* The C ABI used from plain C, with no Python in the process: LayerNorm forward
 * and backward and tanh-GELU forward on the GPU, checked against a double
 * precision computation of the textbook formulas in this file.  Built by gcc as
 * C99 against include/autograd_hip.h and libautograd_hip.so; prints "ok" and
 * exits 0 when every value is within the fp32 tolerance (rtol 1e-5, atol 1e-6;
 * the row-summed dgamma / dbeta within 1e-6 * sqrt(rows) + 2e-6 * |value|).
 *
 * The formulas are those of the reference's independent numpy oracles
 * (layernorm_np and gelu_np, verify_model.py:127-135) and of the LayerNorm
 * gradient it implements in cpu_layernorm_backward (backend.py:435-487). */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include "autograd_hip.h"

#define CHECK(call)                                                              \
    do {                                                                         \
        int rc_ = (call);                                                        \
        if (rc_ != AGRAD_OK) {                                                   \
            fprintf(stderr, "%s -> %d: %s\n", #call, rc_, agrad_last_error());   \
            return 1;                                                            \
        }                                                                        \
    } while (0)

static uint32_t lcg_state = 1333u;
static float next_normalish(void) {
    /* sum of four uniforms, centred: good enough as a test signal */
    double s = 0.0;
    int i;
    for (i = 0; i < 4; ++i) {
        lcg_state = lcg_state * 1664525u + 1013904223u;
        s += (double)(lcg_state >> 8) / 16777216.0;
    }
    return (float)((s - 2.0) * 1.7);
}

static int close_enough(const char* what, const float* got, const double* want, size_t n, double rtol, double atol) {
    size_t i;
    for (i = 0; i < n; ++i) {
        const double err = fabs((double)got[i] - want[i]);
        if (!(err <= atol + rtol * fabs(want[i]))) {
            fprintf(stderr, "%s[%zu]: got %.9g want %.9g\n", what, i, (double)got[i], want[i]);
            return 0;
        }
    }
    return 1;
}

int main(void) {
    const uint64_t rows = 96;
    const uint32_t C = 384;
    const float eps = 1e-5f;
    const size_t n = (size_t)rows * C;
    float *x = malloc(n * 4), *dy = malloc(n * 4), *gamma = malloc(C * 4), *beta = malloc(C * 4);
    float *y = malloc(n * 4), *dx = malloc(n * 4), *act = malloc(n * 4), *dgamma = malloc(C * 4), *dbeta = malloc(C * 4);
    double *wy = malloc(n * 8), *wdx = malloc(n * 8), *wact = malloc(n * 8), *wdg = calloc(C, 8), *wdb = calloc(C, 8);
    agrad_ctx* ctx = NULL;
    uint64_t d_x, d_dy, d_gamma, d_beta, d_y, d_dx, d_act, d_dgamma, d_dbeta, d_ws;
    uint64_t ws_bytes;
    size_t r, c;
    int ok = 1;

    for (r = 0; r < n; ++r) { x[r] = next_normalish(); dy[r] = next_normalish(); }
    for (c = 0; c < C; ++c) { gamma[c] = 1.0f + 0.02f * next_normalish(); beta[c] = 0.02f * next_normalish(); }

    /* expected values, double precision */
    for (r = 0; r < rows; ++r) {
        const float* xr = x + r * C;
        const float* gr = dy + r * C;
        double mean = 0.0, var = 0.0, m1 = 0.0, m2 = 0.0, inv;
        for (c = 0; c < C; ++c) mean += xr[c];
        mean /= C;
        for (c = 0; c < C; ++c) var += (xr[c] - mean) * (xr[c] - mean);
        var /= C;
        inv = 1.0 / sqrt(var + (double)eps);
        for (c = 0; c < C; ++c) {
            const double xh = (xr[c] - mean) * inv, dyg = (double)gr[c] * gamma[c];
            m1 += dyg;
            m2 += dyg * xh;
            wdg[c] += gr[c] * xh;
            wdb[c] += gr[c];
        }
        m1 /= C;
        m2 /= C;
        for (c = 0; c < C; ++c) {
            const double xh = (xr[c] - mean) * inv, dyg = (double)gr[c] * gamma[c];
            const double yv = xh * gamma[c] + beta[c];
            wy[r * C + c] = yv;
            wdx[r * C + c] = inv * (dyg - m1 - xh * m2);
        }
    }
    for (r = 0; r < n; ++r) {
        const double v = x[r];
        wact[r] = 0.5 * v * (1.0 + tanh(0.7978845608028654 * (v + 0.044715 * v * v * v)));
    }

    CHECK(agrad_ctx_create(0, &ctx));
    ws_bytes = agrad_norm_backward_workspace_bytes(rows, C, AGRAD_F32);
    CHECK(agrad_alloc(ctx, n * 4, &d_x));
    CHECK(agrad_alloc(ctx, n * 4, &d_dy));
    CHECK(agrad_alloc(ctx, C * 4, &d_gamma));
    CHECK(agrad_alloc(ctx, C * 4, &d_beta));
    CHECK(agrad_alloc(ctx, n * 4, &d_y));
    CHECK(agrad_alloc(ctx, n * 4, &d_dx));
    CHECK(agrad_alloc(ctx, n * 4, &d_act));
    CHECK(agrad_alloc(ctx, C * 4, &d_dgamma));
    CHECK(agrad_alloc(ctx, C * 4, &d_dbeta));
    CHECK(agrad_alloc(ctx, ws_bytes ? ws_bytes : 16, &d_ws));
    CHECK(agrad_copy_from_host(ctx, d_x, 0, x, n * 4));
    CHECK(agrad_copy_from_host(ctx, d_dy, 0, dy, n * 4));
    CHECK(agrad_copy_from_host(ctx, d_gamma, 0, gamma, C * 4));
    CHECK(agrad_copy_from_host(ctx, d_beta, 0, beta, C * 4));

    /* a buffer id is the device address: typed entry points take it as a pointer */
    CHECK(agrad_norm_forward(ctx, AGRAD_NORM_LAYER, AGRAD_F32, (const void*)(uintptr_t)d_x, NULL,
                             (const float*)(uintptr_t)d_gamma, (const float*)(uintptr_t)d_beta, NULL,
                             (void*)(uintptr_t)d_y, rows, C, eps));
    CHECK(agrad_norm_backward(ctx, AGRAD_NORM_LAYER, AGRAD_F32, (const void*)(uintptr_t)d_x,
                              (const void*)(uintptr_t)d_dy, (const float*)(uintptr_t)d_gamma, NULL,
                              (void*)(uintptr_t)d_dx, NULL, (float*)(uintptr_t)d_dgamma, (float*)(uintptr_t)d_dbeta,
                              (void*)(uintptr_t)d_ws, ws_bytes, rows, C, eps, 0u));
    CHECK(agrad_gelu_forward(ctx, AGRAD_F32, (const void*)(uintptr_t)d_x, (void*)(uintptr_t)d_act, n));
    CHECK(agrad_synchronize(ctx));
    CHECK(agrad_copy_to_host(ctx, d_y, 0, y, n * 4));
    CHECK(agrad_copy_to_host(ctx, d_dx, 0, dx, n * 4));
    CHECK(agrad_copy_to_host(ctx, d_act, 0, act, n * 4));
    CHECK(agrad_copy_to_host(ctx, d_dgamma, 0, dgamma, C * 4));
    CHECK(agrad_copy_to_host(ctx, d_dbeta, 0, dbeta, C * 4));

    ok &= close_enough("layernorm y", y, wy, n, 1e-5, 2e-6);
    ok &= close_enough("layernorm dx", dx, wdx, n, 1e-5, 2e-6);
    ok &= close_enough("gelu y", act, wact, n, 1e-5, 1e-6);
    ok &= close_enough("dgamma", dgamma, wdg, C, 2e-6, 1e-6 * sqrt((double)rows));
    ok &= close_enough("dbeta", dbeta, wdb, C, 2e-6, 1e-6 * sqrt((double)rows));

    /* an error comes back as a status and a message, not as a crash */
    if (agrad_norm_forward(ctx, 7, AGRAD_F32, (const void*)(uintptr_t)d_x, NULL, NULL, NULL, NULL,
                           (void*)(uintptr_t)d_y, rows, C, eps) == AGRAD_OK) {
        fprintf(stderr, "an unknown norm kind was accepted\n");
        ok = 0;
    }
    CHECK(agrad_free(ctx, d_x));
    CHECK(agrad_free(ctx, d_dy));
    CHECK(agrad_free(ctx, d_gamma));
    CHECK(agrad_free(ctx, d_beta));
    CHECK(agrad_free(ctx, d_y));
    CHECK(agrad_free(ctx, d_dx));
    CHECK(agrad_free(ctx, d_act));
    CHECK(agrad_free(ctx, d_dgamma));
    CHECK(agrad_free(ctx, d_dbeta));
    CHECK(agrad_free(ctx, d_ws));
    CHECK(agrad_ctx_destroy(ctx));
    puts(ok ? "ok" : "MISMATCH");
    return ok ? 0 : 1;
}

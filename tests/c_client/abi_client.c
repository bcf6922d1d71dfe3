/*
 * A plain C consumer of libgometal_hip.so: what the cgo preamble of go-metal's cgo_bridge
 * sees.  Allocates one weight / gradient / two state buffers per tensor, runs a few Adam
 * steps through execute_adam_step_mpsgraph and one L-BFGS step with an empty history, and
 * compares every result bit for bit with the CPU checker (oracle/liboracle.so).
 *
 * Exit status: 0 all equal, 1 mismatch or error, 2 no usable GPU (create_metal_device() == 0).
 */
#include "gometal_hip.h"
#include "oracle.h"

#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#define NT 3
static const int kSizes[NT] = {70001, 4096, 33};

static float frand(unsigned *state)          /* xorshift, mapped to (-1, 1) */
{
    unsigned x = *state;
    x ^= x << 13; x ^= x >> 17; x ^= x << 5;
    *state = x;
    return (float)(int)x * (1.0f / 2147483648.0f);
}

static int same_bits(const float *a, const float *b, int n)
{
    return memcmp(a, b, (size_t)n * sizeof(float)) == 0;
}

int main(void)
{
    uintptr_t dev = create_metal_device();
    if (dev == 0) {
        printf("no usable GPU: %s\n", gm_last_error());
        return 2;
    }
    unsigned seed = 12345u;
    float *w[NT], *g[NT], *m[NT], *v[NT], *back = NULL;
    uintptr_t dw[NT], dg[NT], dm[NT], dv[NT];
    int bytes[NT], rc = 0;
    for (int i = 0; i < NT; i++) {
        const int n = kSizes[i];
        bytes[i] = n * (int)sizeof(float);
        w[i] = malloc((size_t)bytes[i]); g[i] = malloc((size_t)bytes[i]);
        m[i] = calloc((size_t)n, sizeof(float)); v[i] = calloc((size_t)n, sizeof(float));
        for (int k = 0; k < n; k++) w[i][k] = 0.02f * frand(&seed);
        dw[i] = allocate_metal_buffer(dev, bytes[i], 1);
        dg[i] = allocate_metal_buffer(dev, bytes[i], 1);
        dm[i] = allocate_metal_buffer(dev, bytes[i], 1);
        dv[i] = allocate_metal_buffer(dev, bytes[i], 1);
        if (!dw[i] || !dg[i] || !dm[i] || !dv[i]) { printf("allocation failed: %s\n", gm_last_error()); return 1; }
        rc |= copy_float32_array_to_metal_buffer(dw[i], w[i], n);
        rc |= zero_metal_buffer(dev, dm[i], bytes[i]);
        rc |= zero_metal_buffer(dev, dv[i], bytes[i]);
    }
    if (rc != 0) { printf("set-up failed: %s\n", gm_last_error()); return 1; }
    back = malloc((size_t)bytes[0]);

    for (int step = 1; step <= 3; step++) {
        for (int i = 0; i < NT; i++) {
            for (int k = 0; k < kSizes[i]; k++) g[i][k] = 0.01f * frand(&seed);
            if (copy_float32_array_to_metal_buffer(dg[i], g[i], kSizes[i]) != 0) return 1;
            gm_oracle_adam_step(w[i], g[i], m[i], v[i], (size_t)kSizes[i], 1e-3f, 0.9f, 0.999f, 1e-8f, 1e-4f, step, 1);
        }
        rc = execute_adam_step_mpsgraph(dev, dw, dg, dm, dv, NT, bytes, 1e-3f, 0.9f, 0.999f, 1e-8f, 1e-4f, step);
        if (rc != 0) { printf("execute_adam_step_mpsgraph: %d (%s)\n", rc, gm_last_error()); return 1; }
    }
    for (int i = 0; i < NT; i++) {
        const float *host[3] = {w[i], m[i], v[i]};
        const uintptr_t devb[3] = {dw[i], dm[i], dv[i]};
        for (int s = 0; s < 3; s++) {
            if (copy_metal_buffer_to_float32_array(devb[s], back, kSizes[i]) != 0) return 1;
            if (!same_bits(back, host[s], kSizes[i])) { printf("Adam: tensor %d stream %d differs\n", i, s); return 1; }
        }
    }

    /* L-BFGS, empty history: w += step * g (cgo_bridge/bridge_optimizer.m:1026-1040, 1219-1250).
     * m / v double as old-gradient / direction buffers, two more lists hold s and y. */
    uintptr_t ds[NT], dy[NT], rho = allocate_metal_buffer(dev, 4, 1), alpha = allocate_metal_buffer(dev, 4, 1);
    for (int i = 0; i < NT; i++) {
        ds[i] = allocate_metal_buffer(dev, bytes[i], 1);
        dy[i] = allocate_metal_buffer(dev, bytes[i], 1);
        if (!ds[i] || !dy[i]) return 1;
    }
    float step_size = 0.0f;
    rc = execute_lbfgs_step_mpsgraph(dev, dw, dg, dm, dv, ds, dy, &rho, alpha, NT, bytes, 1, 0, 0, 0.5f, 1e-4f, 0.9f,
                                     20, 0.0f, 0.0f, &step_size);
    if (rc != 0 || step_size != 0.5f) { printf("execute_lbfgs_step_mpsgraph: %d (%s)\n", rc, gm_last_error()); return 1; }
    for (int i = 0; i < NT; i++) {
        for (int k = 0; k < kSizes[i]; k++) w[i][k] = w[i][k] + 0.5f * g[i][k];
        if (copy_metal_buffer_to_float32_array(dw[i], back, kSizes[i]) != 0) return 1;
        if (!same_bits(back, w[i], kSizes[i])) { printf("L-BFGS: tensor %d differs\n", i); return 1; }
    }

    for (int i = 0; i < NT; i++) {
        deallocate_metal_buffer(dw[i]); deallocate_metal_buffer(dg[i]); deallocate_metal_buffer(dm[i]);
        deallocate_metal_buffer(dv[i]); deallocate_metal_buffer(ds[i]); deallocate_metal_buffer(dy[i]);
        free(w[i]); free(g[i]); free(m[i]); free(v[i]);
    }
    deallocate_metal_buffer(rho);
    deallocate_metal_buffer(alpha);
    free(back);
    destroy_metal_device(dev);
    printf("C client: Adam x3 and one L-BFGS step bit-identical to the CPU checker\n");
    return 0;
}

/*
 * CPU oracle for the L-BFGS step.  TEST INFRASTRUCTURE ONLY (see oracle.h).
 *
 * Restates execute_lbfgs_step_mpsgraph (cgo_bridge/bridge_optimizer.m:980-1321),
 * which is a plain CPU loop nest over unified-memory buffers, statement by
 * statement, including three properties of that code a reader may not expect:
 *   - the recursion starts from q = -g and ends with p = -r (:1025-1038, :1203-1213),
 *     so with an empty or invalid history the weights move by +initial_step * g;
 *   - the newest history slot is part of the two-loop recursion before its y and
 *     rho have been recomputed (the recomputation is step 6, :1242-1312);
 *   - the old gradient is overwritten with the current one (:1237-1238) before
 *     y = g - old_g is formed (:1285-1288), so y is all zeros for finite gradients
 *     and every rho the step itself writes is 0.
 * Every written floating-point operation rounds once to binary32 (build with
 * -ffp-contract=off).
 *
 * Dot products come in two evaluation orders:
 *   GM_ORACLE_DOT_REFERENCE  the reference's: fp32 running sum in element order
 *       (per tensor, tensors then added, for the recursion :1100-1104, :1172-1176;
 *       one running sum across all tensors for s.y, :1294-1297);
 *   GM_ORACLE_DOT_TREE       the HIP library's: exact fp64 products summed by a
 *       fixed radix-1024 tree in fp64, rounded once to fp32 at the end.
 * The tree (same for every dot): each tensor is cut into slices of 1024
 * elements; a node over up to 1024 values v[0..count) is
 *     lane[l] = ((((0.0 + v[l]) + v[l+256]) + v[l+512]) + v[l+768]),  l = 0..255,
 *               terms with index >= count left out,
 *     node    = balanced binary tree over lane[0..255] adding adjacent pairs
 *               (lane[0]+lane[1]) + (lane[2]+lane[3]) ... up to one value.
 * Level 0 applies the node to the products of each slice (slices numbered in
 * tensor order); level k+1 applies it to consecutive groups of 1024 level-k
 * results, until one value is left (no slices: 0.0).
 */
#include "oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#define SLICE 1024
#define LANES 256

static double tree_lanes(double *lane)
{
    for (int width = 1; width < LANES; width *= 2)
        for (int l = 0; l < LANES; l += 2 * width) lane[l] = lane[l] + lane[l + width];
    return lane[0];
}

static double node_of_values(const double *v, size_t count)
{
    double lane[LANES];
    for (int l = 0; l < LANES; l++) {
        double acc = 0.0;
        for (size_t i = (size_t)l; i < count && i < SLICE; i += LANES) acc = acc + v[i];
        lane[l] = acc;
    }
    return tree_lanes(lane);
}

static double node_of_products(const float *a, const float *b, size_t count)
{
    double lane[LANES];
    for (int l = 0; l < LANES; l++) {
        double acc = 0.0;
        for (size_t i = (size_t)l; i < count && i < SLICE; i += LANES)
            acc = acc + (double)a[i] * (double)b[i];      /* the product of two binary32 values is exact in binary64 */
        lane[l] = acc;
    }
    return tree_lanes(lane);
}

static float dot_tree(const float *const *a, const float *const *b, const size_t *n, int num_tensors)
{
    size_t slices = 0;
    for (int t = 0; t < num_tensors; t++) slices += (n[t] + SLICE - 1) / SLICE;
    if (slices == 0) return 0.0f;
    double *cur = (double *)malloc(slices * sizeof(double));
    size_t k = 0;
    for (int t = 0; t < num_tensors; t++)
        for (size_t off = 0; off < n[t]; off += SLICE) {
            const size_t left = n[t] - off;
            cur[k++] = node_of_products(a[t] + off, b[t] + off, left < SLICE ? left : SLICE);
        }
    size_t count = slices;
    while (count > 1) {
        const size_t next = (count + SLICE - 1) / SLICE;
        for (size_t i = 0; i < next; i++) {
            const size_t left = count - i * SLICE;
            cur[i] = node_of_values(cur + i * SLICE, left < SLICE ? left : SLICE);   /* cur[i] is read before it is overwritten: i <= i*SLICE */
        }
        count = next;
    }
    const double total = cur[0];
    free(cur);
    return (float)total;
}

static float dot_reference(const float *const *a, const float *const *b, const size_t *n, int num_tensors,
                           int per_tensor)
{
    float total = 0.0f;
    for (int t = 0; t < num_tensors; t++) {
        if (per_tensor) {
            float dot = 0.0f;                                   /* :1100-1104 */
            for (size_t k = 0; k < n[t]; k++) dot += a[t][k] * b[t][k];
            total += dot;
        } else {
            for (size_t k = 0; k < n[t]; k++) total += a[t][k] * b[t][k];   /* :1294-1297 */
        }
    }
    return total;
}

float gm_oracle_lbfgs_dot(const float *const *a, const float *const *b, const size_t *n, int num_tensors,
                          int dot_mode, int per_tensor)
{
    return dot_mode == GM_ORACLE_DOT_TREE ? dot_tree(a, b, n, num_tensors)
                                          : dot_reference(a, b, n, num_tensors, per_tensor);
}

int gm_oracle_lbfgs_step(float *const *w, const float *const *g, float *const *old_g, float *const *dir,
                         float *const *s, float *const *y, float *rho, float *alpha,
                         const size_t *n, int num_tensors, int history_size, int history_count,
                         int history_index, float initial_step, int dot_mode, float *step_size)
{
    if (num_tensors <= 0 || history_size <= 0 || history_count < 0 || history_count > history_size ||
        history_index < 0 || history_index >= history_size)
        return -5;

    /* step 1, :1025-1038: q = -g */
    for (int i = 0; i < num_tensors; i++)
        for (size_t k = 0; k < n[i]; k++) dir[i][k] = -g[i][k];

    /* step 2, first loop, :1045-1130 */
    for (int j = history_count - 1; j >= 0; j--) {
        const int idx = (history_index - history_count + j + history_size) % history_size;
        const float rho_j = rho[idx];
        if (fabs(rho_j) < 1e-10) {          /* float promoted to double, compared with a double constant */
            alpha[j] = 0.0f;
            continue;
        }
        float alpha_j = gm_oracle_lbfgs_dot((const float *const *)(s + (size_t)idx * num_tensors),
                                            (const float *const *)dir, n, num_tensors, dot_mode, 1);
        alpha_j *= rho_j;
        alpha[j] = alpha_j;
        float *const *yj = y + (size_t)idx * num_tensors;
        for (int i = 0; i < num_tensors; i++)
            for (size_t k = 0; k < n[i]; k++) dir[i][k] = dir[i][k] - alpha_j * yj[i][k];
    }

    /* second loop, :1133-1201 (H0 = identity) */
    for (int j = 0; j < history_count; j++) {
        const int idx = (history_index - history_count + j + history_size) % history_size;
        const float rho_j = rho[idx];
        if (fabs(rho_j) < 1e-10) continue;
        float beta = gm_oracle_lbfgs_dot((const float *const *)(y + (size_t)idx * num_tensors),
                                         (const float *const *)dir, n, num_tensors, dot_mode, 1);
        beta *= rho_j;
        const float coeff = alpha[j] - beta;
        float *const *sj = s + (size_t)idx * num_tensors;
        for (int i = 0; i < num_tensors; i++)
            for (size_t k = 0; k < n[i]; k++) dir[i][k] = dir[i][k] + coeff * sj[i][k];
    }

    /* step 3, :1203-1213: p = -r */
    for (int i = 0; i < num_tensors; i++)
        for (size_t k = 0; k < n[i]; k++) dir[i][k] = -dir[i][k];

    /* step 4, :1215-1216: fixed step */
    const float a = initial_step;
    if (step_size) *step_size = a;

    /* step 5, :1219-1240: x += a * p; old gradient <- current gradient */
    for (int i = 0; i < num_tensors; i++) {
        for (size_t k = 0; k < n[i]; k++) w[i][k] = w[i][k] + a * dir[i][k];
        memcpy(old_g[i], g[i], n[i] * sizeof(float));
    }

    /* step 6, :1242-1312 */
    const int cur = history_index;
    for (int i = 0; i < num_tensors; i++)
        for (size_t k = 0; k < n[i]; k++) s[(size_t)cur * num_tensors + i][k] = a * dir[i][k];

    if (history_count > 0) {
        const int prev = (cur - 1 + history_size) % history_size;
        float *const *yp = y + (size_t)prev * num_tensors;
        float *const *sp = s + (size_t)prev * num_tensors;
        for (int i = 0; i < num_tensors; i++)
            for (size_t k = 0; k < n[i]; k++) yp[i][k] = g[i][k] - old_g[i][k];
        const float s_dot_y = gm_oracle_lbfgs_dot((const float *const *)sp, (const float *const *)yp, n,
                                                  num_tensors, dot_mode, 0);
        rho[prev] = fabs(s_dot_y) > 1e-10 ? 1.0f / s_dot_y : 0.0f;
    }
    return 0;
}

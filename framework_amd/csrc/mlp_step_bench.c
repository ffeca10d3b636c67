/* The README quick-start step (README.md:28-46 of the reference) timed through the engine-level C ABI alone: no
 * language binding between the loop and the library, which is what a Rust `rocm` arm or the N-API shim sees.
 *
 *   x [32,10] ~ U[0,1), Linear(10,64) -> ReLU -> Linear(64,3), crossEntropyLoss on targets in {0,1,2},
 *   backward, Adam{lr 1e-3, beta2 0.95} through clipAndStep (src/optimizer.ts:63-69), gcTensors(keep) per step.
 *
 * usage: mlp_step_bench [fused 0|1] [steps] [warmup]
 * prints one JSON line: ms per step with a wait for the device after every step, ms per step in a loop that only
 * waits at the end, kernel launches per step, and the loss before and after (it must fall). */
#include <stdio.h>
#include <stdlib.h>
#include <stdint.h>
#include <time.h>
#include "mni_rocm.h"

static double now_ms(void) {
    struct timespec t;
    clock_gettime(CLOCK_MONOTONIC, &t);
    return t.tv_sec * 1e3 + t.tv_nsec * 1e-6;
}
static uint64_t rng_state = 0x9e3779b97f4a7c15ull;
static float uniform(float lo, float hi) {
    rng_state ^= rng_state << 13; rng_state ^= rng_state >> 7; rng_state ^= rng_state << 17;
    return lo + (hi - lo) * (float)((rng_state >> 40) & 0xffffff) / 16777216.0f;
}
static uint32_t tensor(const int64_t *shape, int nd, float lo, float hi, int grad) {
    int64_t n = 1;
    for (int i = 0; i < nd; ++i) n *= shape[i];
    float *h = (float *)malloc((size_t)n * sizeof(float));
    for (int64_t i = 0; i < n; ++i) h[i] = uniform(lo, hi);
    const uint32_t id = mni_from_float32(h, (size_t)n, shape, nd);
    free(h);
    if (id == MNI_BAD_ID) { fprintf(stderr, "tensor: %s\n", mni_rocm_last_error()); exit(1); }
    if (grad) mni_set_requires_grad(id, 1);
    return id;
}
#define CHECK_ID(x) do { if ((x) == MNI_BAD_ID) { fprintf(stderr, "%s failed: %s\n", #x, mni_rocm_last_error()); exit(1); } } while (0)

static uint32_t x, w1, b1, w2, b2;
static int64_t targets[32];
static int fused;
static int64_t adam_t;

static uint32_t step(void) {
    const uint32_t params[4] = {w1, b1, w2, b2};
    mni_zero_grad(params, 4);
    uint32_t h, logits;
    if (fused) {
        h = mni_linear(x, w1, b1, MNI_EPI_BIAS_RELU); CHECK_ID(h);
        logits = mni_linear(h, w2, b2, MNI_EPI_BIAS); CHECK_ID(logits);
    } else {
        uint32_t t = mni_matmul(x, w1); CHECK_ID(t);
        t = mni_add(t, b1); CHECK_ID(t);
        h = mni_relu(t); CHECK_ID(h);
        t = mni_matmul(h, w2); CHECK_ID(t);
        logits = mni_add(t, b2); CHECK_ID(logits);
    }
    const int64_t flat[2] = {32, 3};
    const uint32_t v = mni_view(logits, flat, 2); CHECK_ID(v);           /* src/nn.ts:90-100 */
    const uint32_t loss = mni_cross_entropy_loss(v, targets, 32); CHECK_ID(loss);
    if (mni_backward(loss) != MNI_OK) { fprintf(stderr, "backward: %s\n", mni_rocm_last_error()); exit(1); }
    if (mni_clip_and_step(params, 4, 1e-3, 0.9, 0.95, 1e-8, 0.0, ++adam_t, 0.0) < 0) { fprintf(stderr, "step: %s\n", mni_rocm_last_error()); exit(1); }
    return loss;
}
static void collect(void) {
    uint32_t keep[9] = {x, w1, b1, w2, b2};
    size_t n = 5;
    const uint32_t params[4] = {w1, b1, w2, b2};
    for (int i = 0; i < 4; ++i) {
        uint32_t g;
        if (mni_get_grad(params[i], &g) == 1) keep[n++] = g;
    }
    mni_gc_tensors(keep, n);
}

int main(int argc, char **argv) {
    fused = argc > 1 ? atoi(argv[1]) : 1;
    const int steps = argc > 2 ? atoi(argv[2]) : 500, warmup = argc > 3 ? atoi(argv[3]) : 50;
    if (mni_rocm_init(0) != MNI_OK) { fprintf(stderr, "init: %s\n", mni_rocm_last_error()); return 1; }
    const int64_t sx[2] = {32, 10}, sw1[2] = {10, 64}, sb1[1] = {64}, sw2[2] = {64, 3}, sb2[1] = {3};
    x = tensor(sx, 2, 0.f, 1.f, 0);
    w1 = tensor(sw1, 2, -0.316f, 0.316f, 1); b1 = tensor(sb1, 1, -0.316f, 0.316f, 1);
    w2 = tensor(sw2, 2, -0.125f, 0.125f, 1); b2 = tensor(sb2, 1, -0.125f, 0.125f, 1);
    for (int i = 0; i < 32; ++i) targets[i] = (int64_t)(uniform(0.f, 3.f)) % 3;
    double loss_first = 0, loss_last = 0;
    for (int i = 0; i < warmup; ++i) {
        const uint32_t loss = step();
        if (i == 0) mni_get_scalar(loss, &loss_first);
        collect();
    }
    mni_rocm_sync();
    uint64_t launches = 0;
    double t0 = now_ms();
    for (int i = 0; i < steps; ++i) {
        const uint64_t l0 = mni_rocm_launch_count();
        step();
        mni_rocm_sync();
        launches = mni_rocm_launch_count() - l0;
        collect();
    }
    const double ms_sync = (now_ms() - t0) / steps;
    t0 = now_ms();
    for (int i = 0; i < steps; ++i) { step(); collect(); }
    mni_rocm_sync();
    const double ms_loop = (now_ms() - t0) / steps;
    { const uint32_t loss = step(); mni_get_scalar(loss, &loss_last); collect(); }
    printf("{\"fused_linear\": %d, \"steps\": %d, \"ms_per_step_with_a_wait_after_each\": %.5f, \"ms_per_step_in_a_loop\": %.5f, "
           "\"launches_per_step\": %llu, \"loss_first\": %.6f, \"loss_last\": %.6f}\n",
           fused, steps, ms_sync, ms_loop, (unsigned long long)launches, loss_first, loss_last);
    return loss_last < loss_first ? 0 : 2;
}

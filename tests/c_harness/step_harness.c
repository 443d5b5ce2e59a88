/*
 * A caller of libscanet_hip.so that is not Python: plain C99, nothing but include/scanet_hip.h.
 * Builds Dense(8, Sigmoid) >> Dense(3, Softmax) with CategoricalCrossentropy, fills weights and one batch from a
 * 32-bit linear congruential generator, runs three Adam steps (optimizers/Optimizer.scala:136-157) and prints every
 * step's loss and the final parameters.  tests/test_c_harness.py runs it as a child process and compares the
 * printout with the CPU oracle on the same numbers.
 *
 *   gcc -std=c99 -pedantic -Wall -Wextra -Werror -I include tests/c_harness/step_harness.c \
 *       -o tests/c_harness/step_harness -L scanet3_amd -lscanet_hip
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "scanet_hip.h"

#define ROWS 16
#define FEATURES 5
#define HIDDEN 8
#define CLASSES 3
#define STEPS 3

static uint32_t lcg_state = 20251125u;

/* 16 random bits as a float in [0, 1): exact in float32, so any language reproduces it */
static float next_unit(void) {
  lcg_state = lcg_state * 1664525u + 1013904223u;
  return (float)((lcg_state >> 8) & 0xFFFFu) / 65536.0f;
}

#define CHECK(call)                                                              \
  do {                                                                           \
    int rc_ = (call);                                                            \
    if (rc_ != SN_OK) {                                                          \
      fprintf(stderr, "%s failed (%d): %s\n", #call, rc_, sn_last_error());      \
      return 1;                                                                  \
    }                                                                            \
  } while (0)

int main(void) {
  sn_ctx* ctx = NULL;
  sn_model* model = NULL;
  sn_replica* rep = NULL;
  sn_layer_desc layers[6];
  sn_optimizer_desc adam;
  int64_t input_dims[1] = {FEATURES};
  int32_t n_tensors = 0;
  int64_t flat = 0;
  float x[ROWS * FEATURES], y[ROWS * CLASSES];
  void *x_dev = NULL, *y_dev = NULL;
  int i, t;

  memset(layers, 0, sizeof(layers));
  layers[0].kind = SN_LAYER_DENSE;    layers[0].units = HIDDEN;
  layers[1].kind = SN_LAYER_BIAS;     layers[1].units = HIDDEN;
  layers[2].kind = SN_LAYER_ACTIVATE; layers[2].activation = SN_ACT_SIGMOID;
  layers[3].kind = SN_LAYER_DENSE;    layers[3].units = CLASSES;
  layers[4].kind = SN_LAYER_BIAS;     layers[4].units = CLASSES;
  layers[5].kind = SN_LAYER_ACTIVATE; layers[5].activation = SN_ACT_SOFTMAX;
  for (i = 0; i < 6; ++i) layers[i].bn_fused = -1;

  memset(&adam, 0, sizeof(adam));
  adam.kind = SN_OPT_ADAM;            /* Adam.scala:17-22 defaults but the rate */
  adam.rate = 0.05f;
  adam.beta1 = 0.9f;
  adam.beta2 = 0.999f;
  adam.epsilon = 1e-7f;

  CHECK(sn_ctx_create(0, NULL, &ctx));
  CHECK(sn_model_create(ctx, layers, 6, SN_LOSS_CATEGORICAL_CROSSENTROPY, input_dims, 1, ROWS, 0u, &model));
  CHECK(sn_model_param_count(model, &n_tensors, &flat));
  CHECK(sn_replica_create(model, &adam, &rep));

  /* parameters in table order, each value (u - 0.5) / 2 */
  for (i = 0; i < n_tensors; ++i) {
    sn_param_info info;
    float* values;
    int64_t k;
    CHECK(sn_model_param_info(model, i, &info));
    values = (float*)malloc((size_t)info.size * sizeof(float));
    if (!values) return 2;
    for (k = 0; k < info.size; ++k) values[k] = (next_unit() - 0.5f) * 0.5f;
    CHECK(sn_params_set(rep, i, values, info.size));
    free(values);
  }
  for (i = 0; i < ROWS * FEATURES; ++i) x[i] = next_unit();
  memset(y, 0, sizeof(y));
  for (i = 0; i < ROWS; ++i) y[i * CLASSES + (int)(next_unit() * (float)CLASSES)] = 1.0f;

  CHECK(sn_buffer_alloc(ctx, sizeof(x), &x_dev));
  CHECK(sn_buffer_alloc(ctx, sizeof(y), &y_dev));
  CHECK(sn_copy_h2d(ctx, x_dev, x, sizeof(x)));
  CHECK(sn_copy_h2d(ctx, y_dev, y, sizeof(y)));
  CHECK(sn_sync(ctx));

  for (t = 1; t <= STEPS; ++t) {
    float loss = 0.0f;
    CHECK(sn_step(rep, (const float*)x_dev, (const float*)y_dev, ROWS, t, &loss));
    printf("loss %d %.9g\n", t, (double)loss);
  }
  for (i = 0; i < n_tensors; ++i) {
    sn_param_info info;
    float* values;
    int64_t k;
    CHECK(sn_model_param_info(model, i, &info));
    values = (float*)malloc((size_t)info.size * sizeof(float));
    if (!values) return 2;
    CHECK(sn_params_get(rep, i, values, info.size));
    printf("param %s", info.path);
    for (k = 0; k < info.size; ++k) printf(" %.9g", (double)values[k]);
    printf("\n");
    free(values);
  }

  CHECK(sn_buffer_free(ctx, x_dev));
  CHECK(sn_buffer_free(ctx, y_dev));
  CHECK(sn_replica_destroy(rep));
  CHECK(sn_model_destroy(model));
  CHECK(sn_ctx_destroy(ctx));
  return 0;
}

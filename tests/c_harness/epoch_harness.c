/*
 * The calls a JVM binding of libscanet_hip.so makes for one epoch of `Optimizer.run` (optimizers/Optimizer.scala:59-104),
 * from plain C99 with nothing but include/scanet_hip.h: two replicas of Dense(8, Tanh) >> Dense(3, Softmax) start from
 * the same weights, each trains one epoch over its own partition in pinned HOST memory (sn_host_alloc, then
 * sn_train_epoch_host: the TensorIterator -> feed path), the two are averaged (sn_replicas_average: aggregateParams),
 * and the averaged model is read back: its parameters, both Adam slots of the first tensor (sn_optstate_get), its
 * predictions for the first batch (sn_forward into a device buffer) and the accuracy count of that batch
 * (sn_count_correct).  tests/test_c_harness.py runs the program and compares the printout with the CPU oracle.
 *
 *   gcc -std=c99 -pedantic -Wall -Wextra -Werror -I include tests/c_harness/epoch_harness.c \
 *       -o tests/c_harness/epoch_harness -L scanet3_amd -lscanet_hip
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "scanet_hip.h"

#define BATCH 16
#define BATCHES 4            /* full batches per partition */
#define TAIL 5               /* rows of a partial batch behind them, which the epoch skips (optimizers/Iterators.scala:90) */
#define PART_ROWS (BATCH * BATCHES + TAIL)
#define FEATURES 6
#define HIDDEN 8
#define CLASSES 3
#define REPLICAS 2

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

static void print_values(const char* tag, const char* name, const float* v, int64_t n) {
  int64_t k;
  printf("%s %s", tag, name);
  for (k = 0; k < n; ++k) printf(" %.9g", (double)v[k]);
  printf("\n");
}

int main(void) {
  sn_ctx* ctx = NULL;
  sn_model* model = NULL;
  sn_replica* reps[REPLICAS] = {NULL, NULL};
  sn_layer_desc layers[6];
  sn_optimizer_desc adam;
  int64_t input_dims[1] = {FEATURES};
  int32_t n_tensors = 0;
  int64_t flat = 0;
  void* x_host[REPLICAS] = {NULL, NULL};
  void* y_host[REPLICAS] = {NULL, NULL};
  void *x_dev = NULL, *y_dev = NULL, *pred_dev = NULL;
  float pred[BATCH * CLASSES];
  int64_t correct = -1;
  int i, r;

  memset(layers, 0, sizeof(layers));
  layers[0].kind = SN_LAYER_DENSE;    layers[0].units = HIDDEN;
  layers[1].kind = SN_LAYER_BIAS;     layers[1].units = HIDDEN;
  layers[2].kind = SN_LAYER_ACTIVATE; layers[2].activation = SN_ACT_TANH;
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
  CHECK(sn_model_create(ctx, layers, 6, SN_LOSS_CATEGORICAL_CROSSENTROPY, input_dims, 1, BATCH, 0u, &model));
  CHECK(sn_model_param_count(model, &n_tensors, &flat));
  for (r = 0; r < REPLICAS; ++r) CHECK(sn_replica_create(model, &adam, &reps[r]));

  /* the broadcast: every replica starts the epoch from the same weights (Optimizer.scala:72-73), each value (u - 0.5) / 2 */
  for (i = 0; i < n_tensors; ++i) {
    sn_param_info info;
    float* values;
    int64_t k;
    CHECK(sn_model_param_info(model, i, &info));
    values = (float*)malloc((size_t)info.size * sizeof(float));
    if (!values) return 2;
    for (k = 0; k < info.size; ++k) values[k] = (next_unit() - 0.5f) * 0.5f;
    for (r = 0; r < REPLICAS; ++r) CHECK(sn_params_set(reps[r], i, values, info.size));
    free(values);
  }

  /* one partition per replica in pinned host memory: all of x first, then the labels */
  for (r = 0; r < REPLICAS; ++r) {
    float *xp, *yp;
    CHECK(sn_host_alloc(ctx, sizeof(float) * PART_ROWS * FEATURES, &x_host[r]));
    CHECK(sn_host_alloc(ctx, sizeof(float) * PART_ROWS * CLASSES, &y_host[r]));
    xp = (float*)x_host[r];
    yp = (float*)y_host[r];
    for (i = 0; i < PART_ROWS * FEATURES; ++i) xp[i] = next_unit();
    memset(yp, 0, sizeof(float) * PART_ROWS * CLASSES);
    for (i = 0; i < PART_ROWS; ++i) yp[i * CLASSES + (int)(next_unit() * (float)CLASSES)] = 1.0f;
  }

  /* optimizeOnPartition on every partition (Optimizer.scala:106-161), then aggregateParams (:196-230) */
  for (r = 0; r < REPLICAS; ++r) {
    int32_t iterations = 0;
    float loss = 0.0f;
    CHECK(sn_train_epoch_host(reps[r], (const float*)x_host[r], (const float*)y_host[r], PART_ROWS, BATCH, 0, &iterations, &loss));
    printf("epoch %d %d %.9g\n", r, (int)iterations, (double)loss);
  }
  CHECK(sn_replicas_average(reps, REPLICAS));

  /* what the driver reads back: the averaged model from either replica */
  for (r = 0; r < REPLICAS; ++r) {
    for (i = 0; i < n_tensors; ++i) {
      sn_param_info info;
      float* values;
      char tag[16];
      CHECK(sn_model_param_info(model, i, &info));
      values = (float*)malloc((size_t)info.size * sizeof(float));
      if (!values) return 2;
      CHECK(sn_params_get(reps[r], i, values, info.size));
      sprintf(tag, "param%d", r);
      print_values(tag, info.path, values, info.size);
      if (i == 0) {
        int slot;
        for (slot = 0; slot < 2; ++slot) {
          CHECK(sn_optstate_get(reps[r], i, slot, values, info.size));
          sprintf(tag, "slot%d_%d", slot, r);
          print_values(tag, info.path, values, info.size);
        }
      }
      free(values);
    }
  }

  /* TrainedModel.result / accuracy on the first batch of partition 0 (estimators/package.scala:18-48) */
  CHECK(sn_buffer_alloc(ctx, sizeof(float) * BATCH * FEATURES, &x_dev));
  CHECK(sn_buffer_alloc(ctx, sizeof(float) * BATCH * CLASSES, &y_dev));
  CHECK(sn_buffer_alloc(ctx, sizeof(float) * BATCH * CLASSES, &pred_dev));
  CHECK(sn_copy_h2d(ctx, x_dev, x_host[0], sizeof(float) * BATCH * FEATURES));
  CHECK(sn_copy_h2d(ctx, y_dev, y_host[0], sizeof(float) * BATCH * CLASSES));
  CHECK(sn_forward(reps[0], (const float*)x_dev, BATCH, (float*)pred_dev));
  CHECK(sn_copy_d2h(ctx, pred, pred_dev, sizeof(pred)));
  print_values("pred", "batch0", pred, BATCH * CLASSES);
  CHECK(sn_count_correct(reps[0], (const float*)x_dev, (const float*)y_dev, BATCH, &correct));
  printf("correct %ld\n", (long)correct);

  CHECK(sn_buffer_free(ctx, x_dev));
  CHECK(sn_buffer_free(ctx, y_dev));
  CHECK(sn_buffer_free(ctx, pred_dev));
  for (r = 0; r < REPLICAS; ++r) {
    CHECK(sn_host_free(ctx, x_host[r]));
    CHECK(sn_host_free(ctx, y_host[r]));
    CHECK(sn_replica_destroy(reps[r]));
  }
  CHECK(sn_model_destroy(model));
  CHECK(sn_ctx_destroy(ctx));
  return 0;
}

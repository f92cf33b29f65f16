/* A compiled host driving the C ABI directly, the way Knet's Julia code does through ccall: one forward + backward step of the
 * MLP of examples/mnist-mlp/mlp.jl:25-35 (784-64-10, batch 100), every device operation an entry point of knet8.h.
 *
 *   mlp_step IN OUT [steps]        (IN may be "@random")
 *
 * IN holds, as raw little-endian data in this order: float W1[64*784], b1[64], W2[10*64], b2[10], x[784*100] (all column-major),
 * int32 labels[100] (1-based).  OUT receives float loss, dW1[64*784], db1[64], dW2[10*64], db2[10].  With `steps` the step is then
 * repeated that many times on a stream without host synchronisation and the rate is printed ("steps_per_sec N"), then captured
 * into a graph and replayed as often ("graph_steps_per_sec N").
 * Test infrastructure: the parity test compares OUT with the CPU oracle. */
#include <stdio.h>
#include <stdlib.h>
#include <time.h>
#include "knet8.h"

enum { D0 = 784, D1 = 64, D2 = 10, NB = 100 };

static float *dev(size_t n) {
  float *p = (float *)knet8_malloc(n * sizeof(float));
  if (!p) { fprintf(stderr, "knet8_malloc failed: %s\n", knet8_last_error()); exit(2); }
  return p;
}

static void up(void *d, const void *h, size_t bytes) {
  if (knet8_memcpy(d, h, bytes, 1, 0) != 0) { fprintf(stderr, "upload failed\n"); exit(2); }
}

struct net {
  float *W1, *b1, *W2, *b2, *x, *y1, *mean, *db2, *dW2, *dy1, *db1, *dW1;
  int *labels;
};

static void step(struct net *n, hipStream_t st) {
  /* hidden layer forward: y1 = relu(W1*x .+ b1) */
  gemm_bias_act_32_stream('N', 'N', D1, NB, D0, 1.0f, n->W1, D1, n->x, D0, n->b1, 1, n->y1, D1, st);
  /* output layer, forward and backward in one launch: s = W2*y1 .+ b2 (kept inside the kernel), the mean loss, ds = (softmax(s) - onehot)/NB,
   * dW2 = ds*y1', db2, dy1 = W2'*ds; then the hidden layer's backward: dz1 = relu'(y1).*dy1, dW1, db1.
   * (These entry points return 1 for layers outside the range of their kernel; these are not.) */
  if (dense_head_32_stream(D2, NB, D1, n->W2, n->b2, n->y1, n->labels, 1.0f / NB, n->dW2, n->db2, n->dy1, NULL, n->mean, NULL, st) != 0 ||
      dense_back_32_stream(1, D1, NB, D0, n->W1, n->x, n->y1, n->dy1, n->dW1, n->db1, NULL, st) != 0) {
    fprintf(stderr, "dense_back declined or failed\n");
    exit(4);
  }
}

int main(int argc, char **argv) {
  if (argc < 3) { fprintf(stderr, "usage: %s IN OUT [steps]\n", argv[0]); return 2; }
  const long steps = argc > 3 ? atol(argv[3]) : 0;
  const size_t nW1 = (size_t)D1 * D0, nW2 = (size_t)D2 * D1, nx = (size_t)D0 * NB;
  const size_t nin = nW1 + D1 + nW2 + D2 + nx;
  float *h = (float *)malloc(nin * sizeof(float));
  int hl[NB];
  FILE *f = NULL;
  if (argv[1][0] == '@') { /* "@random": inputs from a fixed linear congruential sequence, for profiling runs without an input file */
    unsigned long long sd = 88172645463325252ULL;
    for (size_t i = 0; i < nin; i++) { sd = sd * 6364136223846793005ULL + 1442695040888963407ULL; h[i] = ((float)(sd >> 40) / 16777216.0f - 0.5f) * 0.1f; }
    for (int i = 0; i < NB; i++) { sd = sd * 6364136223846793005ULL + 1442695040888963407ULL; hl[i] = 1 + (int)((sd >> 33) % D2); }
  } else {
    f = fopen(argv[1], "rb");
    if (!f || fread(h, sizeof(float), nin, f) != nin || fread(hl, sizeof(int), NB, f) != NB) { fprintf(stderr, "cannot read %s\n", argv[1]); return 2; }
    fclose(f);
  }
  if (knet8_device_count() < 1) { fprintf(stderr, "no device\n"); return 3; }
  struct net n;
  n.W1 = dev(nW1); n.b1 = dev(D1); n.W2 = dev(nW2); n.b2 = dev(D2); n.x = dev(nx);
  n.y1 = dev(D1 * NB); n.mean = dev(1);
  n.db2 = dev(D2); n.dW2 = dev(nW2); n.dy1 = dev(D1 * NB); n.db1 = dev(D1); n.dW1 = dev(nW1);
  n.labels = (int *)knet8_malloc(NB * sizeof(int));
  const float *p = h;
  up(n.W1, p, nW1 * 4); p += nW1;
  up(n.b1, p, D1 * 4); p += D1;
  up(n.W2, p, nW2 * 4); p += nW2;
  up(n.b2, p, D2 * 4); p += D2;
  up(n.x, p, nx * 4);
  up(n.labels, hl, NB * sizeof(int));

  hipStream_t st = knet8_stream_create();
  step(&n, st);
  float loss = 0.0f;
  if (knet8_memcpy(&loss, n.mean, sizeof(float), 2, st) != 0) { fprintf(stderr, "download failed\n"); return 2; } /* blocks */
  const char *err = knet8_last_error();
  if (err) { fprintf(stderr, "libknet8: %s\n", err); return 4; }

  const size_t nout = 1 + nW1 + D1 + nW2 + D2;
  float *o = (float *)malloc(nout * sizeof(float));
  float *q = o;
  *q++ = loss;
  knet8_memcpy(q, n.dW1, nW1 * 4, 2, st); q += nW1;
  knet8_memcpy(q, n.db1, D1 * 4, 2, st); q += D1;
  knet8_memcpy(q, n.dW2, nW2 * 4, 2, st); q += nW2;
  knet8_memcpy(q, n.db2, D2 * 4, 2, st);
  f = fopen(argv[2], "wb");
  if (!f || fwrite(o, sizeof(float), nout, f) != nout) { fprintf(stderr, "cannot write %s\n", argv[2]); return 2; }
  fclose(f);

  if (steps > 0) {
    for (int i = 0; i < 20; i++) step(&n, st);
    knet8_synchronize(st);
    struct timespec t0, t1;
    clock_gettime(CLOCK_MONOTONIC, &t0);
    for (long i = 0; i < steps; i++) step(&n, st);
    knet8_synchronize(st);
    clock_gettime(CLOCK_MONOTONIC, &t1);
    const double dt = (double)(t1.tv_sec - t0.tv_sec) + 1e-9 * (double)(t1.tv_nsec - t0.tv_nsec);
    printf("steps_per_sec %.1f\n", (double)steps / dt);
    err = knet8_last_error();
    if (err) { fprintf(stderr, "libknet8: %s\n", err); return 4; }
    /* the same step captured once into a graph and replayed */
    if (knet8_graph_begin(st) != 0) { fprintf(stderr, "capture failed: %s\n", knet8_last_error()); return 4; }
    step(&n, st);
    void *g = knet8_graph_end(st);
    if (!g) { fprintf(stderr, "capture failed: %s\n", knet8_last_error()); return 4; }
    for (int i = 0; i < 20; i++) knet8_graph_launch(g, st);
    knet8_synchronize(st);
    clock_gettime(CLOCK_MONOTONIC, &t0);
    for (long i = 0; i < steps; i++) knet8_graph_launch(g, st);
    knet8_synchronize(st);
    clock_gettime(CLOCK_MONOTONIC, &t1);
    const double dg = (double)(t1.tv_sec - t0.tv_sec) + 1e-9 * (double)(t1.tv_nsec - t0.tv_nsec);
    printf("graph_steps_per_sec %.1f\n", (double)steps / dg);
    knet8_graph_destroy(g);
    err = knet8_last_error();
    if (err) { fprintf(stderr, "libknet8: %s\n", err); return 4; }
  }
  knet8_stream_destroy(st);
  return 0;
}

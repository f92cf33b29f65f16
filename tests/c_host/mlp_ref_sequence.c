/* The launch sequence an UNCHANGED Knet model emits for one forward + backward step of the MLP of examples/mnist-mlp/mlp.jl:25-35
 * (784-64-10, batch 100), issued by a compiled host through entry points that carry the reference's own names and meanings only:
 *
 *   forward   predict (mlp.jl:25-33):  gemm, add_32_12 (the .+ of the (m,1) bias), relu_32, gemm, add_32_12
 *             nll (src/ops20/loss.jl:37-41): logsoftmax_32 (the cudnnSoftmaxForward call of src/ops20_gpu/softmax.jl:47), upload of the
 *             linear indices findindices computes on the host (loss.jl:116-140), getents_32 (getindex, src/knetarrays/getindex.jl:217-220),
 *             sum_32_20 (blocking: the loss comes back to the host)
 *   backward  what AutoGrad's sweep emits for that tape: fill_32 (the -1/N of the mean), fill_32 + addents_32 (ungetindex into a zero
 *             (C,N) array, src/autograd_gpu/getindex.jl:5-18, addto.jl:59-65), logsoftmaxback_32 (cudnnSoftmaxBackward, softmax.jl:54),
 *             sum_32_21 (unbroadcast of the bias, src/knetarrays/reduction.jl:21-77), gemm NT and TN (src/knetarrays/linalg.jl:11-18),
 *             reluback_32_11, sum_32_21, gemm NT
 * 18 kernel launches, one host-to-device and one device-to-host copy per step.  No fused entry point, no graph.
 *
 *   mlp_ref_sequence IN OUT [steps [own_product_mflop]]     (IN may be "@random")
 *
 * IN / OUT as for mlp_step.c: float W1[64*784], b1[64], W2[10*64], b2[10], x[784*100] column-major, int32 labels[100] (1-based) in;
 * float loss, dW1, db1, dW2, db2 out.  With `steps` the step is repeated and "steps_per_sec N" printed.  `own_product_mflop` > 0 sets
 * knet8_tune key 3 (products up to that size on the library's own kernels); by default every product goes to hipBLASLt.
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

static void up(void *d, const void *h, size_t bytes, hipStream_t st) {
  if (knet8_memcpy(d, h, bytes, 1, st) != 0) { fprintf(stderr, "upload failed\n"); exit(2); }
}

struct net {
  float *W1, *b1, *W2, *b2, *x;
  float *z1, *a1, *y1, *z2, *s2, *lp, *picked, *dpicked, *dlp, *dz2, *db2, *dW2, *dy1, *dz1, *db1, *dW1;
  int *ents;
  int hl[NB], hents[NB];
};

static float step(struct net *n, hipStream_t st) {
  /* forward */
  gemm_32_stream('N', 'N', D1, NB, D0, 1.0f, n->W1, D1, n->x, D0, 0.0f, n->z1, D1, st);
  add_32_12_stream(D1 * NB, n->z1, 1, D1 * NB, n->b1, 1, D1, n->a1, st);
  relu_32_stream(D1 * NB, n->a1, n->y1, st);
  gemm_32_stream('N', 'N', D2, NB, D1, 1.0f, n->W2, D2, n->y1, D1, 0.0f, n->z2, D2, st);
  add_32_12_stream(D2 * NB, n->z2, 1, D2 * NB, n->b2, 1, D2, n->s2, st);
  logsoftmax_32_stream(D2, NB, n->s2, n->lp, st);
  for (int j = 0; j < NB; j++) n->hents[j] = j * D2 + n->hl[j];   /* findindices, dims=1: (j-1)*C + label_j, 1-based */
  up(n->ents, n->hents, NB * sizeof(int), st);
  getents_32_stream(NB, n->ents, n->lp, n->picked, st);
  const float loss = -sum_32_20_stream(NB, n->picked, st) / (float)NB;
  /* backward */
  fill_32_stream(NB, -1.0f / (float)NB, n->dpicked, st);
  fill_32_stream(D2 * NB, 0.0f, n->dlp, st);
  addents_32_stream(NB, n->ents, n->dlp, n->dpicked, st);
  logsoftmaxback_32_stream(D2, NB, n->lp, n->dlp, n->dz2, st);
  sum_32_21_stream(D2 * NB, n->dz2, 1, D2, n->db2, st);
  gemm_32_stream('N', 'T', D2, D1, NB, 1.0f, n->dz2, D2, n->y1, D1, 0.0f, n->dW2, D2, st);
  gemm_32_stream('T', 'N', D1, NB, D2, 1.0f, n->W2, D2, n->dz2, D2, 0.0f, n->dy1, D1, st);
  reluback_32_11_stream(D1 * NB, n->dy1, n->y1, n->dz1, st);
  sum_32_21_stream(D1 * NB, n->dz1, 1, D1, n->db1, st);
  gemm_32_stream('N', 'T', D1, D0, NB, 1.0f, n->dz1, D1, n->x, D0, 0.0f, n->dW1, D1, st);
  return loss;
}

int main(int argc, char **argv) {
  if (argc < 3) { fprintf(stderr, "usage: %s IN OUT [steps [own_product_mflop]]\n", argv[0]); return 2; }
  const long steps = argc > 3 ? atol(argv[3]) : 0;
  const int own = argc > 4 ? atoi(argv[4]) : 0;
  const size_t nW1 = (size_t)D1 * D0, nW2 = (size_t)D2 * D1, nx = (size_t)D0 * NB;
  const size_t nin = nW1 + D1 + nW2 + D2 + nx;
  float *h = (float *)malloc(nin * sizeof(float));
  struct net n;
  if (argv[1][0] == '@') {
    unsigned long long sd = 88172645463325252ULL;
    for (size_t i = 0; i < nin; i++) { sd = sd * 6364136223846793005ULL + 1442695040888963407ULL; h[i] = ((float)(sd >> 40) / 16777216.0f - 0.5f) * 0.1f; }
    for (int i = 0; i < NB; i++) { sd = sd * 6364136223846793005ULL + 1442695040888963407ULL; n.hl[i] = 1 + (int)((sd >> 33) % D2); }
  } else {
    FILE *f = fopen(argv[1], "rb");
    if (!f || fread(h, sizeof(float), nin, f) != nin || fread(n.hl, sizeof(int), NB, f) != NB) { fprintf(stderr, "cannot read %s\n", argv[1]); return 2; }
    fclose(f);
  }
  if (knet8_device_count() < 1) { fprintf(stderr, "no device\n"); return 3; }
  if (own > 0) knet8_tune(3, own);
  hipStream_t st = knet8_stream_create();
  n.W1 = dev(nW1); n.b1 = dev(D1); n.W2 = dev(nW2); n.b2 = dev(D2); n.x = dev(nx);
  n.z1 = dev(D1 * NB); n.a1 = dev(D1 * NB); n.y1 = dev(D1 * NB); n.z2 = dev(D2 * NB); n.s2 = dev(D2 * NB); n.lp = dev(D2 * NB);
  n.picked = dev(NB); n.dpicked = dev(NB); n.dlp = dev(D2 * NB); n.dz2 = dev(D2 * NB); n.db2 = dev(D2); n.dW2 = dev(nW2);
  n.dy1 = dev(D1 * NB); n.dz1 = dev(D1 * NB); n.db1 = dev(D1); n.dW1 = dev(nW1);
  n.ents = (int *)knet8_malloc(NB * sizeof(int));
  const float *p = h;
  up(n.W1, p, nW1 * 4, st); p += nW1;
  up(n.b1, p, D1 * 4, st); p += D1;
  up(n.W2, p, nW2 * 4, st); p += nW2;
  up(n.b2, p, D2 * 4, st); p += D2;
  up(n.x, p, nx * 4, st);

  const float loss = step(&n, st);
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
  FILE *f = fopen(argv[2], "wb");
  if (!f || fwrite(o, sizeof(float), nout, f) != nout) { fprintf(stderr, "cannot write %s\n", argv[2]); return 2; }
  fclose(f);

  if (steps > 0) {
    for (int i = 0; i < 20; i++) step(&n, st);
    knet8_synchronize(st);
    struct timespec t0, t1;
    clock_gettime(CLOCK_MONOTONIC, &t0);
    float acc = 0.0f;
    for (long i = 0; i < steps; i++) acc += step(&n, st);
    knet8_synchronize(st);
    clock_gettime(CLOCK_MONOTONIC, &t1);
    const double dt = (double)(t1.tv_sec - t0.tv_sec) + 1e-9 * (double)(t1.tv_nsec - t0.tv_nsec);
    printf("steps_per_sec %.1f\n", (double)steps / dt);
    printf("mean_loss %.6f\n", (double)acc / (double)steps);
    err = knet8_last_error();
    if (err) { fprintf(stderr, "libknet8: %s\n", err); return 4; }
  }
  knet8_stream_destroy(st);
  return 0;
}

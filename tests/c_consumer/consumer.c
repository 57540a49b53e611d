/*
 * A consumer of include/gorgonia_hip.h written in plain C99: what a cgo (or
 * any other FFI) binding does, without C++ and without Python in the way.
 * It fills a gh_cmd[] for a small forward pass
 *
 *   conv 3x3 (+Rectify in the epilogue) -> MaxPool2D 2x2/2 -> product with a
 *   weight matrix (+bias row) -> SoftMax,   and   sigmoid(a * b) elementwise
 *
 * hands the whole array to ONE gh_submit, waits once, and writes every result
 * to a file for the test to compare byte for byte with the same commands
 * submitted through the ctypes binding.
 *
 *   consumer <in.bin> <out.bin>
 *
 * in.bin : float32 x[B,C,H,W] w[F,C,3,3] wd[F*PH*PW,NO] bias[NO] a[NE] b[NE]
 * out.bin: float32 conv[B,F,H,W] pool[B,F,PH,PW] prob[B,NO] e[NE]
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "gorgonia_hip.h"

enum { B = 4, C = 3, H = 12, W = 12, F = 8, PH = 6, PW = 6, NO = 10, NE = 1000 };
enum { NX = B * C * H * W, NW = F * C * 9, NWD = F * PH * PW * NO, NCONV = B * F * H * W, NPOOL = B * F * PH * PW, NPROB = B * NO };

static gh_ctx* ctx;

static void die(const char* what, int rc) {
  char msg[512];
  msg[0] = 0;
  if (ctx) gh_last_error(ctx, msg, (int)sizeof msg);
  fprintf(stderr, "consumer: %s failed with code %d: %s\n", what, rc, msg);
  exit(1);
}

#define CHECK(call) do { int rc_ = (call); if (rc_ != GH_OK) die(#call, rc_); } while (0)

static gh_devptr dev_floats(size_t n, const float* init) {
  gh_devptr p = 0;
  CHECK(gh_malloc(ctx, (int64_t)(n * sizeof(float)), &p));
  if (init) CHECK(gh_memcpy_h2d(ctx, p, init, (int64_t)(n * sizeof(float))));
  return p;
}

int main(int argc, char** argv) {
  static float in[NX + NW + NWD + NO + 2 * NE];
  static float out[NCONV + NPOOL + NPROB + NE];
  const size_t n_in = sizeof in / sizeof in[0], n_out = sizeof out / sizeof out[0];
  const float *x = in, *w = x + NX, *wd = w + NW, *bias = wd + NWD, *a = bias + NO, *b = a + NE;
  gh_devptr dx, dw, dwd, dbias, da, db, dconv, dpool, dlogit, dprob, de;
  gh_cmd cmd[6];
  gh_cmd* c;
  FILE* f;
  int n = 0;

  if (argc != 3) {
    fprintf(stderr, "usage: %s in.bin out.bin\n", argv[0]);
    return 2;
  }
  f = fopen(argv[1], "rb");
  if (!f || fread(in, sizeof(float), n_in, f) != n_in) {
    fprintf(stderr, "consumer: cannot read %lu floats from %s\n", (unsigned long)n_in, argv[1]);
    return 2;
  }
  fclose(f);

  CHECK(gh_init(0, 0, &ctx));
  dx = dev_floats(NX, x);
  dw = dev_floats(NW, w);
  dwd = dev_floats(NWD, wd);
  dbias = dev_floats(NO, bias);
  da = dev_floats(NE, a);
  db = dev_floats(NE, b);
  dconv = dev_floats(NCONV, NULL);
  dpool = dev_floats(NPOOL, NULL);
  dlogit = dev_floats(NPROB, NULL);
  dprob = dev_floats(NPROB, NULL);
  de = dev_floats(NE, NULL);

  memset(cmd, 0, sizeof cmd);

  c = &cmd[n++]; /* convolution_cuda.go:95-121 with the Rectify that follows it */
  c->opcode = GH_OP_CONV2D;
  c->flags = GH_FLAG_ACT_RELU;
  c->ptr[0] = dx; c->ptr[1] = dw; c->ptr[2] = dconv;
  c->dim[0] = B; c->dim[1] = C; c->dim[2] = H; c->dim[3] = W; c->dim[4] = F;
  c->dim[5] = 3; c->dim[6] = 3;
  c->dim[7] = 1; c->dim[8] = 1;
  c->dim[9] = 1; c->dim[10] = 1;
  c->dim[11] = 1; c->dim[12] = 1;

  c = &cmd[n++]; /* maxpool_cuda.go:94-111 */
  c->opcode = GH_OP_MAXPOOL2D;
  c->ptr[0] = dconv; c->ptr[1] = dpool;
  c->dim[0] = B; c->dim[1] = F; c->dim[2] = H; c->dim[3] = W;
  c->dim[4] = 2; c->dim[5] = 2;
  c->dim[10] = 2; c->dim[11] = 2;

  c = &cmd[n++]; /* cuda/linalg.go:110: (B x F*PH*PW) * (F*PH*PW x NO), bias row added */
  c->opcode = GH_OP_GEMM;
  c->flags = GH_FLAG_GEMM_BIAS;
  c->ptr[0] = dpool; c->ptr[1] = dwd; c->ptr[2] = dlogit; c->ptr[3] = dbias;
  c->dim[0] = B; c->dim[1] = NO; c->dim[2] = F * PH * PW;
  c->dim[3] = F * PH * PW; c->dim[4] = NO; c->dim[5] = NO;

  c = &cmd[n++]; /* op_softmax.go:99-128 */
  c->opcode = GH_OP_SOFTMAX;
  c->ptr[0] = dlogit; c->ptr[1] = dprob;
  c->dim[0] = B; c->dim[1] = NO;

  c = &cmd[n++]; /* elembinop.mul_vv_f32 into a third buffer */
  c->opcode = GH_OP_ELEM_BIN;
  c->flags = GH_FLAG_FN(GH_MUL) | GH_FLAG_MODE(GH_VV) | GH_FLAG_DTYPE(GH_F32);
  c->ptr[0] = da; c->ptr[1] = db; c->ptr[2] = de;
  c->dim[0] = NE;

  c = &cmd[n++]; /* elemunaryop.sigmoid_f32 in place */
  c->opcode = GH_OP_ELEM_UNARY;
  c->flags = GH_FLAG_FN(GH_SIGMOID) | GH_FLAG_DTYPE(GH_F32);
  c->ptr[0] = de;
  c->dim[0] = NE;

  {
    char msg[256];
    int rc = gh_validate(cmd, n, msg, (int)sizeof msg);
    if (rc != GH_OK) {
      fprintf(stderr, "consumer: gh_validate: %s\n", msg);
      return 1;
    }
  }
  CHECK(gh_submit(ctx, cmd, n)); /* the one crossing for the whole segment */
  CHECK(gh_memcpy_d2h(ctx, out, dconv, (int64_t)(NCONV * sizeof(float))));
  CHECK(gh_memcpy_d2h(ctx, out + NCONV, dpool, (int64_t)(NPOOL * sizeof(float))));
  CHECK(gh_memcpy_d2h(ctx, out + NCONV + NPOOL, dprob, (int64_t)(NPROB * sizeof(float))));
  CHECK(gh_memcpy_d2h(ctx, out + NCONV + NPOOL + NPROB, de, (int64_t)(NE * sizeof(float))));
  CHECK(gh_sync(ctx));

  /* a command the engine has no function for is refused, nothing runs */
  cmd[0].opcode = GH_OP__COUNT;
  if (gh_submit(ctx, cmd, 1) == GH_OK) {
    fprintf(stderr, "consumer: an unknown opcode was accepted\n");
    return 1;
  }
  CHECK(gh_clear_error(ctx));

  CHECK(gh_free(ctx, dx)); CHECK(gh_free(ctx, dw)); CHECK(gh_free(ctx, dwd)); CHECK(gh_free(ctx, dbias));
  CHECK(gh_free(ctx, da)); CHECK(gh_free(ctx, db)); CHECK(gh_free(ctx, dconv)); CHECK(gh_free(ctx, dpool));
  CHECK(gh_free(ctx, dlogit)); CHECK(gh_free(ctx, dprob)); CHECK(gh_free(ctx, de));
  CHECK(gh_close(ctx));
  ctx = NULL;

  f = fopen(argv[2], "wb");
  if (!f || fwrite(out, sizeof(float), n_out, f) != n_out) {
    fprintf(stderr, "consumer: cannot write %s\n", argv[2]);
    return 2;
  }
  fclose(f);
  printf("consumer: %d commands in one gh_submit, %lu floats written (%s)\n", n, (unsigned long)n_out, gh_version());
  return 0;
}

/* A caller of libmlora.so that knows nothing of Python or PyTorch: plain C over the HIP runtime API and
 * include/mlora.h, the way a binding written in any language would drive the C ABI.
 *
 *   cabi_gpu_check IN OUT
 *
 * IN  : int64 header[12] = {T, h_in, h_out, n_adapters, max_rank, n_slots, dtype, slot, a_loc_len, rows_a,
 *       rows_b, 0}, then ids[T], a_start[A], a_len[A], a_loc[a_loc_len] (int64), then 16-bit arrays scales[A],
 *       x[T*h_in], y[T*h_out], key_buffer[rows_a*h_in], value_buffer[rows_b*h_out].
 * OUT : 16-bit arrays y_plan[T*h_out]  (mlora_tile_lookup + mlora_build_plan + mlora_lora_apply),
 *       delta[T*max_rank]              (mlora_dispatch_bgmv, shrink direction, plan = NULL),
 *       y_bgmv[T*h_out]                (mlora_dispatch_bgmv, expand direction, on that delta).
 * The test that runs this program compares OUT with the oracle.  Exit status 0 = every call succeeded.
 *
 * The calls follow valora/csrc/lora_ops.cc:76-126 (dispatch_bgmv) and the per-layer call pattern of
 * valora/models/peft/lora_unordered_batch_infer.py:946-988. */
#include <hip/hip_runtime_api.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include "mlora.h"

#define HIP(call)                                                                              \
  do {                                                                                         \
    hipError_t e_ = (call);                                                                    \
    if (e_ != hipSuccess) {                                                                    \
      fprintf(stderr, "%s:%d: %s: %s\n", __FILE__, __LINE__, #call, hipGetErrorString(e_));    \
      return 2;                                                                                \
    }                                                                                          \
  } while (0)
#define MLORA(call)                                                                            \
  do {                                                                                         \
    int rc_ = (call);                                                                          \
    if (rc_ != 0) {                                                                            \
      fprintf(stderr, "%s:%d: %s -> %d: %s\n", __FILE__, __LINE__, #call, rc_, mlora_last_error()); \
      return 3;                                                                                \
    }                                                                                          \
  } while (0)

static void *read_array(FILE *f, size_t bytes) {
  void *p = malloc(bytes ? bytes : 1);
  if (!p || fread(p, 1, bytes, f) != bytes) {
    fprintf(stderr, "short input file\n");
    exit(4);
  }
  return p;
}

static int to_device(void **dev, const void *host, size_t bytes) {
  HIP(hipMalloc(dev, bytes ? bytes : 16));
  HIP(hipMemcpy(*dev, host, bytes, hipMemcpyHostToDevice));
  return 0;
}

int main(int argc, char **argv) {
  if (argc != 3) {
    fprintf(stderr, "usage: %s IN OUT\n", argv[0]);
    return 1;
  }
  FILE *f = fopen(argv[1], "rb");
  if (!f) {
    perror(argv[1]);
    return 1;
  }
  int64_t h[12];
  if (fread(h, sizeof(int64_t), 12, f) != 12) return 4;
  const int64_t T = h[0], h_in = h[1], h_out = h[2], A = h[3], R = h[4], a_loc_len = h[8], rows_a = h[9], rows_b = h[10];
  const int32_t n_slots = (int32_t)h[5], slot = (int32_t)h[7];
  const mlora_dtype dt = h[6] == 0 ? MLORA_F16 : MLORA_BF16;
  int64_t *ids = read_array(f, (size_t)T * 8), *a_start = read_array(f, (size_t)A * 8), *a_len = read_array(f, (size_t)A * 8);
  int64_t *a_loc = read_array(f, (size_t)a_loc_len * 8);
  uint16_t *scales = read_array(f, (size_t)A * 2), *x = read_array(f, (size_t)(T * h_in) * 2);
  uint16_t *y0 = read_array(f, (size_t)(T * h_out) * 2);
  uint16_t *kbuf = read_array(f, (size_t)(rows_a * h_in) * 2), *vbuf = read_array(f, (size_t)(rows_b * h_out) * 2);
  fclose(f);

  HIP(hipSetDevice(0));
  hipStream_t st;
  HIP(hipStreamCreate(&st));
  void *d_ids, *d_start, *d_len, *d_loc, *d_scales, *d_x, *d_y, *d_y2, *d_k, *d_v, *d_delta;
  if (to_device(&d_ids, ids, (size_t)T * 8) || to_device(&d_start, a_start, (size_t)A * 8) ||
      to_device(&d_len, a_len, (size_t)A * 8) || to_device(&d_loc, a_loc, (size_t)a_loc_len * 8) ||
      to_device(&d_scales, scales, (size_t)A * 2) || to_device(&d_x, x, (size_t)(T * h_in) * 2) ||
      to_device(&d_y, y0, (size_t)(T * h_out) * 2) || to_device(&d_y2, y0, (size_t)(T * h_out) * 2) ||
      to_device(&d_k, kbuf, (size_t)(rows_a * h_in) * 2) || to_device(&d_v, vbuf, (size_t)(rows_b * h_out) * 2))
    return 2;
  HIP(hipMalloc(&d_delta, (size_t)(T * R) * 2 + 16));
  HIP(hipMemset(d_delta, 0, (size_t)(T * R) * 2));

  mlora_pool pa = {d_k, rows_a, d_start, d_len, d_loc, A, a_loc_len, n_slots};
  mlora_pool pb = {d_v, rows_b, d_start, d_len, d_loc, A, a_loc_len, n_slots};

  /* ---- the planned op: one plan for the batch, then shrink + expand of one target */
  mlora_tile_config cfg;
  MLORA(mlora_tile_lookup(T, R, h_in, A, &cfg));
  mlora_plan plan = {0};
  plan.bytes = mlora_plan_bytes(T, A);
  HIP(hipMalloc(&plan.dev, plan.bytes));
  MLORA(mlora_build_plan(st, &plan, d_ids, T, d_start, d_len, A, n_slots, cfg.bm_shrink, cfg.bm_expand));
  size_t scratch_bytes = mlora_scratch_bytes(T, R, cfg.ksplit > 0 ? cfg.ksplit : 1);
  if (cfg.flags & MLORA_ONE_LAUNCH) {
    const size_t one = mlora_one_launch_scratch_bytes(T, A, R, cfg.ksplit, 1);
    if (one > scratch_bytes) scratch_bytes = one;
  }
  void *scratch;
  HIP(hipMalloc(&scratch, scratch_bytes));
  MLORA(mlora_lora_apply(st, &plan, scratch, scratch_bytes, d_y, d_x, T, h_in, h_out, R, &pa, &pb, slot, d_scales,
                         cfg.ksplit, cfg.flags, dt));

  /* ---- the reference's entry point, two calls, no plan: delta = shrink(x); y += expand(delta) */
  const size_t ws_bytes = mlora_workspace_bytes(T, A, R);
  void *ws;
  HIP(hipMalloc(&ws, ws_bytes));
  MLORA(mlora_dispatch_bgmv(st, d_delta, d_x, &pa, d_ids, slot, d_scales, T, h_in, R, dt, ws, ws_bytes, NULL));
  MLORA(mlora_dispatch_bgmv(st, d_y2, d_delta, &pb, d_ids, slot, d_scales, T, R, h_out, dt, ws, ws_bytes, NULL));
  HIP(hipStreamSynchronize(st));

  uint16_t *out = malloc((size_t)(T * h_out) * 2 + 2);
  uint16_t *dl = malloc((size_t)(T * R) * 2 + 2);
  FILE *o = fopen(argv[2], "wb");
  if (!o || !out || !dl) return 1;
  HIP(hipMemcpy(out, d_y, (size_t)(T * h_out) * 2, hipMemcpyDeviceToHost));
  fwrite(out, 2, (size_t)(T * h_out), o);
  HIP(hipMemcpy(dl, d_delta, (size_t)(T * R) * 2, hipMemcpyDeviceToHost));
  fwrite(dl, 2, (size_t)(T * R), o);
  HIP(hipMemcpy(out, d_y2, (size_t)(T * h_out) * 2, hipMemcpyDeviceToHost));
  fwrite(out, 2, (size_t)(T * h_out), o);
  fclose(o);
  printf("cabi_gpu_check: T=%lld %lld->%lld adapters=%lld tile=(%d,%d,%d,flags %d) ok\n", (long long)T, (long long)h_in,
         (long long)h_out, (long long)A, cfg.bm_shrink, cfg.ksplit, cfg.bm_expand, cfg.flags);
  return 0;
}

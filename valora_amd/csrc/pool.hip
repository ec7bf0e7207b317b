// Adapter residency for gfx950: the row allocator of the paged pool, the row scatter / gather that
// moves an adapter's weights between its packed form and its pool rows, and the re-indexing of
// a_start / a_len / a_loc / a_scaling when adapters are dropped.
//
// Reference behaviour (all of it PyTorch tensor code and one Triton copy kernel there):
//   * first-fit row allocation, contiguous allocation, free   valora/common/mem_allocator.py:30-75,203-217
//   * key_buffer[layer][loc] = w_combined[0], value_buffer[layer][loc] = w_combined[1] per layer
//                                                  valora/server/router/model_infer/infer_adapter.py:45-91
//   * offload: free the rows of dropped adapters, rebuild the index tensors, copy the surviving
//     a_loc segments                               infer_adapter.py:176-256, var_len_copy :263-284
//
// Everything here is byte / integer work and is bit-exact with that behaviour.  The allocator
// state is one byte per pool row (1 = free), the layout of the reference's torch.bool tensor.
#include "kernel_common.h"

namespace mlora {

namespace {

constexpr int POOL_THREADS = 1024;
constexpr int POOL_WAVES = POOL_THREADS / 64;

// exclusive scan of one int per thread over the workgroup; *total = sum.  scratch: POOL_WAVES ints.
__device__ __forceinline__ int wg_exclusive_scan(int v, int *total, int *scratch) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int inc = v;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int o = __shfl_up(inc, d, 64);
    if (lane >= d) inc += o;
  }
  __syncthreads();   // scratch may still be read from an earlier call
  if (lane == 63) scratch[wave] = inc;
  __syncthreads();
  int before = 0, sum = 0;
#pragma unroll
  for (int w = 0; w < POOL_WAVES; ++w) {
    const int s = scratch[w];
    if (w < wave) before += s;
    sum += s;
  }
  *total = sum;
  return before + inc - v;
}

__device__ __forceinline__ int wg_max(int v, int *scratch) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) v = max(v, __shfl_xor(v, d, 64));
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  int m = scratch[0];
#pragma unroll
  for (int w = 1; w < POOL_WAVES; ++w) m = max(m, scratch[w]);
  return m;
}

__device__ __forceinline__ int wg_min(int v, int *scratch) { return -wg_max(-v, scratch); }

constexpr int ITEMS = 16;   // pool rows per thread per pass (one 16-byte load of the state)

// First fit: the first `need` free rows in index order are handed out and marked taken
// (mem_allocator.py:35-56: cumsum of the state, select cumsum <= need && free).
// status[0] = rows granted, status[1] = free rows seen before the scan stopped.
__global__ __launch_bounds__(POOL_THREADS) void pool_alloc_kernel(uint8_t *__restrict__ state, int64_t tot,
                                                                   int64_t need, int64_t *__restrict__ out,
                                                                   int32_t *__restrict__ status) {
  __shared__ int scratch[POOL_WAVES];
  const int tid = threadIdx.x;
  int64_t granted = 0;
  for (int64_t base = 0; base < tot && granted < need; base += (int64_t)POOL_THREADS * ITEMS) {
    const int64_t i0 = base + (int64_t)tid * ITEMS;
    uint8_t st[ITEMS];
    int nfree = 0;
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
      st[k] = (i0 + k < tot) ? state[i0 + k] : (uint8_t)0;
      nfree += st[k] != 0;
    }
    int total;
    int rank = wg_exclusive_scan(nfree, &total, scratch);
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
      if (st[k] != 0) {
        const int64_t pos = granted + rank;
        if (pos < need) {
          out[pos] = i0 + k;
          state[i0 + k] = 0;
        }
        ++rank;
      }
    }
    granted += total;
  }
  if (tid == 0) {
    status[0] = (int32_t)(granted < need ? granted : need);
    status[1] = (int32_t)(granted > 0x7fffffff ? 0x7fffffff : granted);
  }
}

// First run of `need` consecutive free rows (mem_allocator.py:59-75).  status[0] = first row of
// the run, or -1 when there is none (the reference returns None and leaves the state untouched).
__global__ __launch_bounds__(POOL_THREADS) void pool_alloc_contiguous_kernel(uint8_t *__restrict__ state,
                                                                              int64_t tot, int64_t need,
                                                                              int64_t *__restrict__ out,
                                                                              int32_t *__restrict__ status) {
  __shared__ int scratch[POOL_WAVES];
  __shared__ int s_carry;
  const int tid = threadIdx.x;
  // a window [i-need+1, i] is free iff the last taken row at or before i is < i-need+1
  int carry = -1;           // last taken row seen in earlier passes
  int found = 0x7fffffff;   // end row i of the first free window
  for (int64_t base = 0; base < tot && found == 0x7fffffff; base += (int64_t)POOL_THREADS * ITEMS) {
    const int i0 = (int)(base + (int64_t)tid * ITEMS);
    uint8_t st[ITEMS];
    int last_local = -1;
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
      st[k] = (i0 + k < tot) ? state[i0 + k] : (uint8_t)0;   // rows past the end count as taken
      if (st[k] == 0) last_local = i0 + k;
    }
    // inclusive max-scan of last_local over the threads, made exclusive
    const int lane = tid & 63, wave = tid >> 6;
    int inc = last_local;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int o = __shfl_up(inc, d, 64);
      if (lane >= d) inc = max(inc, o);
    }
    __syncthreads();
    if (lane == 63) scratch[wave] = inc;
    __syncthreads();
    int before = carry;
    for (int w = 0; w < wave; ++w) before = max(before, scratch[w]);
    int prev = __shfl_up(inc, 1, 64);
    if (lane == 0) prev = -1;
    int last = max(before, prev);     // last taken row strictly before this thread's rows
    int mine = 0x7fffffff;
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
      const int i = i0 + k;
      if (st[k] == 0) last = i;
      else if (i < tot && (int64_t)i - last >= need && mine == 0x7fffffff) mine = i;
    }
    if (tid == POOL_THREADS - 1) s_carry = max(before, inc);
    found = wg_min(mine, scratch);    // has barriers: s_carry is visible afterwards
    carry = s_carry;
  }
  if (found != 0x7fffffff) {
    const int64_t start = (int64_t)found - need + 1;
    for (int64_t k = tid; k < need; k += POOL_THREADS) {
      out[k] = start + k;
      state[start + k] = 0;
    }
    if (tid == 0) status[0] = (int32_t)start;
  } else if (tid == 0) {
    status[0] = -1;
  }
}

// state[index[i]] = 1 (mem_allocator.py:203-217); rows outside the pool are ignored
__global__ __launch_bounds__(256) void pool_free_kernel(uint8_t *__restrict__ state, int64_t tot,
                                                         const int64_t *__restrict__ index, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) {
    const int64_t row = index[i];
    if (row >= 0 && row < tot) state[row] = 1;
  }
}

__global__ __launch_bounds__(256) void pool_fill_kernel(uint8_t *__restrict__ state, int64_t tot, int value) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < tot) state[i] = (uint8_t)value;
}

// Row scatter / gather between a packed matrix [layers][n][row_bytes] and pool rows
// [layers][pool_rows][row_bytes]:  SCATTER  pool[l][loc[i]] = packed[l][i]
//                                  GATHER   packed[l][i]   = pool[l][loc[i]]
// One workgroup copies RPW rows of one layer with 16-byte accesses; pure HBM traffic
// (2 * row_bytes per row).  Rows whose loc is outside the pool are skipped (gather: zero filled).
constexpr int RPW = 4;
template <bool SCATTER>
__global__ __launch_bounds__(256) void pool_rows_kernel(unsigned char *__restrict__ pool, int64_t pool_rows,
                                                         int64_t pool_layer_stride, unsigned char *__restrict__ packed,
                                                         int64_t packed_layer_stride, const int64_t *__restrict__ loc,
                                                         int64_t n, int64_t row_bytes) {
  const int layer = blockIdx.y;
  const int64_t vec_per_row = row_bytes >> 4;
  unsigned char *pl = pool + (int64_t)layer * pool_layer_stride;
  unsigned char *pk = packed + (int64_t)layer * packed_layer_stride;
  const u32x4 *src[RPW];
  u32x4 *dst[RPW];
  bool live[RPW], fill[RPW];
#pragma unroll
  for (int k = 0; k < RPW; ++k) {
    const int64_t i = (int64_t)blockIdx.x * RPW + k;
    const int64_t row = i < n ? loc[i] : -1;
    const bool ok = row >= 0 && row < pool_rows;
    u32x4 *prow = reinterpret_cast<u32x4 *>(pl + (ok ? row : 0) * row_bytes);
    u32x4 *krow = reinterpret_cast<u32x4 *>(pk + (i < n ? i : 0) * row_bytes);
    src[k] = SCATTER ? krow : prow;
    dst[k] = SCATTER ? prow : krow;
    live[k] = ok;                        // copy this row
    fill[k] = !SCATTER && i < n && !ok;  // gather of a row outside the pool: zeros
  }
  // all loads of a pass are issued before the first store
  for (int64_t v = threadIdx.x; v < vec_per_row; v += 256) {
    u32x4 t[RPW];
#pragma unroll
    for (int k = 0; k < RPW; ++k) t[k] = live[k] ? src[k][v] : u32x4{0, 0, 0, 0};
#pragma unroll
    for (int k = 0; k < RPW; ++k)
      if (live[k] || fill[k]) dst[k][v] = t[k];
  }
}

// Re-indexing after adapters were dropped (infer_adapter.py:228-251).  keep[] = surviving old
// adapter indices, ascending.  One workgroup: new_len / new_scaling gathered, new_start = their
// exclusive running sum.
__global__ __launch_bounds__(POOL_THREADS) void index_compact_kernel(
    const int32_t *__restrict__ keep, int n_keep, int n_old, const int64_t *__restrict__ old_len,
    const uint16_t *__restrict__ old_scaling, int64_t *__restrict__ new_start, int64_t *__restrict__ new_len,
    uint16_t *__restrict__ new_scaling, int32_t *__restrict__ status) {
  __shared__ int scratch[POOL_WAVES];
  const int tid = threadIdx.x;
  int64_t carry = 0;
  int bad = 0;
  for (int base = 0; base < n_keep; base += POOL_THREADS) {
    const int i = base + tid;
    int len = 0;
    if (i < n_keep) {
      const int a = keep[i];
      if (a >= 0 && a < n_old) {
        const int64_t l = old_len[a];
        len = (l < 0 || l > 0x3fffff) ? 0 : (int)l;
        new_len[i] = old_len[a];
        new_scaling[i] = old_scaling[a];
      } else {
        bad = 1;
        new_len[i] = 0;
        new_scaling[i] = 0;
      }
    }
    int total;
    const int before = wg_exclusive_scan(len, &total, scratch);
    if (i < n_keep) new_start[i] = carry + before;
    carry += total;
  }
  bad = wg_max(bad, scratch);
  if (tid == 0) {
    status[0] = bad;                       // 1: an index of keep[] was outside [0, n_old)
    status[1] = (int32_t)(carry > 0x7fffffff ? 0x7fffffff : carry);   // entries of the new a_loc
  }
}

// new_loc[new_start[i] + j] = old_loc[old_start[keep[i]] + j]   (var_len_copy, infer_adapter.py:263-284);
// one workgroup per surviving adapter
__global__ __launch_bounds__(256) void index_copy_loc_kernel(const int32_t *__restrict__ keep, int n_old,
                                                              const int64_t *__restrict__ old_start,
                                                              const int64_t *__restrict__ old_len,
                                                              const int64_t *__restrict__ old_loc, int64_t old_loc_len,
                                                              const int64_t *__restrict__ new_start,
                                                              int64_t *__restrict__ new_loc, int64_t new_loc_len) {
  const int a = keep[blockIdx.x];
  if (a < 0 || a >= n_old) return;
  const int64_t src = old_start[a], dst = new_start[blockIdx.x];
  const int64_t len = min(old_len[a], old_loc_len);   // a corrupt length must not turn into a long loop
  for (int64_t j = threadIdx.x; j < len; j += 256)
    if (src + j >= 0 && src + j < old_loc_len && dst + j < new_loc_len) new_loc[dst + j] = old_loc[src + j];
}

// frees the pool rows of every adapter that is NOT in keep[] (ascending): workgroup g handles the
// old indices between keep[g-1] and keep[g]
__global__ __launch_bounds__(256) void index_free_dropped_kernel(const int32_t *__restrict__ keep, int n_keep,
                                                                  int n_old, const int64_t *__restrict__ old_start,
                                                                  const int64_t *__restrict__ old_len,
                                                                  const int64_t *__restrict__ old_loc,
                                                                  int64_t old_loc_len, uint8_t *__restrict__ state,
                                                                  int64_t tot) {
  const int g = blockIdx.x;   // 0 .. n_keep
  const int lo = g == 0 ? 0 : keep[g - 1] + 1;
  const int hi = g == n_keep ? n_old : keep[g];
  for (int a = max(lo, 0); a < min(hi, n_old); ++a) {
    const int64_t src = old_start[a];
    const int64_t len = min(old_len[a], old_loc_len);
    for (int64_t j = threadIdx.x; j < len; j += 256) {
      if (src + j < 0 || src + j >= old_loc_len) continue;
      const int64_t row = old_loc[src + j];
      if (row >= 0 && row < tot) state[row] = 1;
    }
  }
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int rows_call(bool scatter, hipStream_t st, void *pool, int64_t pool_rows, int64_t pool_layer_stride, void *packed,
              int64_t packed_layer_stride, const int64_t *loc, int64_t n, int64_t row_bytes, int32_t n_layers) {
  const char *who = scatter ? "pool_scatter_rows" : "pool_gather_rows";
  if (n < 0 || pool_rows < 0 || n_layers < 0 || row_bytes <= 0)
    return fail(MLORA_ERR_INVALID, "%s: negative size", who);
  if (n == 0 || n_layers == 0) return MLORA_OK;
  if (!pool || !packed || !loc) return fail(MLORA_ERR_INVALID, "%s: null pointer", who);
  if ((row_bytes & 15) || (pool_layer_stride & 15) || (packed_layer_stride & 15) || !aligned16(pool) ||
      !aligned16(packed))
    return fail(MLORA_ERR_INVALID, "%s: rows and layer strides must be multiples of 16 bytes and 16-byte aligned", who);
  if (n_layers > 65535) return fail(MLORA_ERR_INVALID, "%s: more than 65535 layers", who);
  const int64_t blocks = (n + RPW - 1) / RPW;
  if (blocks > 0x7fffffff) return fail(MLORA_ERR_INVALID, "%s: too many rows", who);
  dim3 grid((unsigned)blocks, (unsigned)n_layers);
  if (scatter)
    hipLaunchKernelGGL(pool_rows_kernel<true>, grid, dim3(256), 0, st, static_cast<unsigned char *>(pool), pool_rows,
                       pool_layer_stride, static_cast<unsigned char *>(packed), packed_layer_stride, loc, n, row_bytes);
  else
    hipLaunchKernelGGL(pool_rows_kernel<false>, grid, dim3(256), 0, st, static_cast<unsigned char *>(pool), pool_rows,
                       pool_layer_stride, static_cast<unsigned char *>(packed), packed_layer_stride, loc, n, row_bytes);
  return check_launch(who);
}

}  // namespace

}  // namespace mlora

using namespace mlora;

extern "C" {

int mlora_pool_alloc(void *stream, void *mem_state, int64_t tot_size, int64_t need, int64_t *out_index,
                     int32_t *status) {
  if (tot_size < 0 || need < 0 || tot_size > (1 << 30))
    return fail(MLORA_ERR_INVALID, "pool_alloc: tot_size=%lld need=%lld out of range", (long long)tot_size,
                (long long)need);
  if (!status || (tot_size > 0 && !mem_state) || (need > 0 && !out_index))
    return fail(MLORA_ERR_INVALID, "pool_alloc: null pointer");
  if (need > tot_size)
    return fail(MLORA_ERR_WORKSPACE, "warn no enough pool space: need_size %lld left_size at most %lld",
                (long long)need, (long long)tot_size);
  hipLaunchKernelGGL(pool_alloc_kernel, dim3(1), dim3(POOL_THREADS), 0, (hipStream_t)stream,
                     static_cast<uint8_t *>(mem_state), tot_size, need, out_index, status);
  return check_launch("pool_alloc_kernel");
}

int mlora_pool_alloc_contiguous(void *stream, void *mem_state, int64_t tot_size, int64_t need, int64_t *out_index,
                                int32_t *status) {
  if (tot_size < 0 || need <= 0 || tot_size > (1 << 30))
    return fail(MLORA_ERR_INVALID, "pool_alloc_contiguous: tot_size=%lld need=%lld out of range", (long long)tot_size,
                (long long)need);
  if (!status || !mem_state || !out_index) return fail(MLORA_ERR_INVALID, "pool_alloc_contiguous: null pointer");
  if (need > tot_size)
    return fail(MLORA_ERR_WORKSPACE, "warn no enough pool space: need_size %lld left_size at most %lld",
                (long long)need, (long long)tot_size);
  hipLaunchKernelGGL(pool_alloc_contiguous_kernel, dim3(1), dim3(POOL_THREADS), 0, (hipStream_t)stream,
                     static_cast<uint8_t *>(mem_state), tot_size, need, out_index, status);
  return check_launch("pool_alloc_contiguous_kernel");
}

int mlora_pool_free(void *stream, void *mem_state, int64_t tot_size, const int64_t *index, int64_t n) {
  if (tot_size < 0 || n < 0) return fail(MLORA_ERR_INVALID, "pool_free: negative size");
  if (n == 0) return MLORA_OK;
  if (!mem_state || !index) return fail(MLORA_ERR_INVALID, "pool_free: null pointer");
  hipLaunchKernelGGL(pool_free_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     static_cast<uint8_t *>(mem_state), tot_size, index, n);
  return check_launch("pool_free_kernel");
}

int mlora_pool_fill(void *stream, void *mem_state, int64_t tot_size, int32_t is_free) {
  if (tot_size < 0) return fail(MLORA_ERR_INVALID, "pool_fill: negative size");
  if (tot_size == 0) return MLORA_OK;
  if (!mem_state) return fail(MLORA_ERR_INVALID, "pool_fill: null pointer");
  hipLaunchKernelGGL(pool_fill_kernel, dim3((unsigned)((tot_size + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     static_cast<uint8_t *>(mem_state), tot_size, is_free ? 1 : 0);
  return check_launch("pool_fill_kernel");
}

int mlora_pool_scatter_rows(void *stream, void *pool, int64_t pool_rows, int64_t pool_layer_stride_bytes,
                            const void *packed, int64_t packed_layer_stride_bytes, const int64_t *loc, int64_t n,
                            int64_t row_bytes, int32_t n_layers) {
  return rows_call(true, (hipStream_t)stream, pool, pool_rows, pool_layer_stride_bytes, const_cast<void *>(packed),
                   packed_layer_stride_bytes, loc, n, row_bytes, n_layers);
}

int mlora_pool_gather_rows(void *stream, const void *pool, int64_t pool_rows, int64_t pool_layer_stride_bytes,
                           void *packed, int64_t packed_layer_stride_bytes, const int64_t *loc, int64_t n,
                           int64_t row_bytes, int32_t n_layers) {
  return rows_call(false, (hipStream_t)stream, const_cast<void *>(pool), pool_rows, pool_layer_stride_bytes, packed,
                   packed_layer_stride_bytes, loc, n, row_bytes, n_layers);
}

int mlora_index_compact(void *stream, const int32_t *keep, int32_t n_keep, int32_t n_old, const int64_t *old_start,
                        const int64_t *old_len, const int64_t *old_loc, int64_t old_loc_len, const void *old_scaling,
                        int64_t *new_start, int64_t *new_len, int64_t *new_loc, int64_t new_loc_len, void *new_scaling,
                        void *mem_state, int64_t tot_size, int32_t *status) {
  if (n_keep < 0 || n_old < 0 || n_keep > n_old || old_loc_len < 0 || new_loc_len < 0 || tot_size < 0)
    return fail(MLORA_ERR_INVALID, "index_compact: n_keep=%d n_old=%d out of range", n_keep, n_old);
  if (n_old > MAX_ADAPTERS) return fail(MLORA_ERR_NO_KERNEL, "index_compact: more than %lld adapters", (long long)MAX_ADAPTERS);
  if (!status) return fail(MLORA_ERR_INVALID, "index_compact: status is null");
  if (n_old == 0) return MLORA_OK;
  if (!old_start || !old_len || !old_scaling || (old_loc_len > 0 && !old_loc))
    return fail(MLORA_ERR_INVALID, "index_compact: null old index tensor");
  if (n_keep > 0 && (!keep || !new_start || !new_len || !new_scaling || (new_loc_len > 0 && !new_loc)))
    return fail(MLORA_ERR_INVALID, "index_compact: null new index tensor");
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL(index_compact_kernel, dim3(1), dim3(POOL_THREADS), 0, st, keep, n_keep, n_old, old_len,
                     static_cast<const uint16_t *>(old_scaling), new_start, new_len,
                     static_cast<uint16_t *>(new_scaling), status);
  if (int rc = check_launch("index_compact_kernel")) return rc;
  if (n_keep > 0) {
    hipLaunchKernelGGL(index_copy_loc_kernel, dim3((unsigned)n_keep), dim3(256), 0, st, keep, n_old, old_start, old_len,
                       old_loc, old_loc_len, new_start, new_loc, new_loc_len);
    if (int rc = check_launch("index_copy_loc_kernel")) return rc;
  }
  if (mem_state) {
    hipLaunchKernelGGL(index_free_dropped_kernel, dim3((unsigned)(n_keep + 1)), dim3(256), 0, st, keep, n_keep, n_old,
                       old_start, old_len, old_loc, old_loc_len, static_cast<uint8_t *>(mem_state), tot_size);
    if (int rc = check_launch("index_free_dropped_kernel")) return rc;
  }
  return MLORA_OK;
}

}  // extern "C"

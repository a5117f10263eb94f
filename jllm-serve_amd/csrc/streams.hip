// Several residual streams per row (hyper-connections), a norm without statistics (Dynamic Tanh), and a table row added
// by index. Everything here is element by element in fp32: no sums over a row, so a row's result depends on nothing
// but the row. The streams of a row lie side by side, x [rows, S, width] fp32.
//
//   gather_add     x[t, :] += table[ids[t], :]                        (a learned position table at the input)
//   dyntanh_read   u[c] = sum_s in[s] x[t', s, c] (in == null: the row itself, S = 1; t' = rows ? rows[t] : t);
//                  out[t, k, c] = tanh(alpha u[c]) w[c] + b[c] for k < copies, in the output's type (a sublayer's input
//                  read from the streams; the embedding's norm written once per stream; the final norm of the
//                  streams' sum over the wanted rows)
//   streams_write  all streams at once from the old ones: new[r] = sum_s mix[s, r] old[s] + outw[r] y, in place; and,
//                  with next_in, the next sublayer's input from the new streams in the same pass:
//                  out[t, c] = tanh(alpha sum_r next_in[r] new[r][c]) w[c] + b[c]
#include <math.h>

#include "common.h"

#define ST_THREADS 256
#define ST_MAX_STREAMS 16

template <typename T>
__global__ __launch_bounds__(ST_THREADS) void gather_add_kernel(float* __restrict__ x, int ldx, const T* __restrict__ table,
                                                                const int* __restrict__ ids, int width, int table_rows) {
  const int t = blockIdx.x;
  const size_t row = (size_t)min(max(ids[t], 0), table_rows - 1) * width;  // the host refuses indices beyond the table
  float* o = x + (size_t)t * ldx;
  for (int i = threadIdx.x; i < width; i += ST_THREADS) o[i] += ldf(table, row + i);
}

extern "C" int jllm_gather_add(float* x, int ldx, const void* table, int table_dtype, int table_rows, const int* ids, int n,
                               int width, hipStream_t stream) {
  if (n <= 0) return 0;
  if (width <= 0 || ldx < width || table_rows <= 0) JLLM_FAIL("gather_add: rows of %d in a stride of %d, a table of %d rows", width, ldx, table_rows);
  JLLM_DISPATCH_1(table_dtype, T, {
    gather_add_kernel<T><<<n, ST_THREADS, 0, stream>>>(x, ldx, (const T*)table, ids, width, table_rows);
  })
  JLLM_CHECK_LAUNCH("gather_add");
  return 0;
}

// ---------------------------------------------------------------------------------------------------------------------

__device__ __forceinline__ float dyn_tanh(float u, float alpha, float w, float b) { return fmaf(tanhf(alpha * u), w, b); }

template <typename TO>
__global__ __launch_bounds__(ST_THREADS) void dyntanh_read_kernel(const float* __restrict__ x, const int* __restrict__ rows,
                                                                  int width, int S, const float* __restrict__ in_w,
                                                                  const float* __restrict__ w, const float* __restrict__ b,
                                                                  const float* __restrict__ alpha, TO* __restrict__ out, int ldo,
                                                                  int copies) {
  const int t = blockIdx.x;
  const float* xr = x + (size_t)(rows ? rows[t] : t) * S * width;
  const float a = alpha[0];
  float iw[ST_MAX_STREAMS];
#pragma unroll
  for (int s = 0; s < ST_MAX_STREAMS; ++s) iw[s] = (in_w && s < S) ? in_w[s] : 1.0f;
  for (int c = threadIdx.x; c < width; c += ST_THREADS) {
    float u;
    if (in_w) {
      u = 0.f;
#pragma unroll
      for (int s = 0; s < ST_MAX_STREAMS; ++s)
        if (s < S) u = fmaf(iw[s], xr[(size_t)s * width + c], u);
    } else {
      u = xr[c];
    }
    const float v = dyn_tanh(u, a, w[c], b[c]);
    for (int k = 0; k < copies; ++k) stf(out + (size_t)t * ldo, (size_t)k * width + c, v);
  }
}

extern "C" int jllm_dyntanh_read(const float* x, const int* rows, int n, int width, int S, const float* in_w, const float* w,
                                 const float* b, const float* alpha, void* out, int out_dtype, int ldo, int copies,
                                 hipStream_t stream) {
  if (n <= 0) return 0;
  if (width <= 0 || S < 1 || S > ST_MAX_STREAMS || copies < 1 || ldo < copies * width)
    JLLM_FAIL("dyntanh_read: width %d, %d streams (1..%d are taken), %d copies in rows of %d", width, S, ST_MAX_STREAMS, copies, ldo);
  if (!in_w && S != 1) JLLM_FAIL("dyntanh_read: %d streams need their weights", S);
  if (!w || !b || !alpha) JLLM_FAIL("dyntanh_read: the norm has a weight, a bias and a slope");
  JLLM_DISPATCH_1(out_dtype, TO, {
    dyntanh_read_kernel<TO><<<n, ST_THREADS, 0, stream>>>(x, rows, width, S, in_w, w, b, alpha, (TO*)out, ldo, copies);
  })
  JLLM_CHECK_LAUNCH("dyntanh_read");
  return 0;
}

// ---------------------------------------------------------------------------------------------------------------------

template <typename TO>
__global__ __launch_bounds__(ST_THREADS) void streams_write_kernel(float* __restrict__ x, const float* __restrict__ y, int ldy,
                                                                   int width, int S, const float* __restrict__ mix,
                                                                   const float* __restrict__ outw,
                                                                   const float* __restrict__ next_in, const float* __restrict__ w,
                                                                   const float* __restrict__ b, const float* __restrict__ alpha,
                                                                   TO* __restrict__ out, int ldo) {
  __shared__ float m[ST_MAX_STREAMS * ST_MAX_STREAMS + 2 * ST_MAX_STREAMS];
  float* ow = m + ST_MAX_STREAMS * ST_MAX_STREAMS;
  float* ni = ow + ST_MAX_STREAMS;
  if (threadIdx.x < S * S) m[threadIdx.x] = mix[threadIdx.x];
  if (threadIdx.x < S) {
    ow[threadIdx.x] = outw[threadIdx.x];
    ni[threadIdx.x] = next_in ? next_in[threadIdx.x] : 0.f;
  }
  __syncthreads();
  const int t = blockIdx.x;
  float* xr = x + (size_t)t * S * width;
  const float a = next_in ? alpha[0] : 0.f;
  for (int c = threadIdx.x; c < width; c += ST_THREADS) {
    float old[ST_MAX_STREAMS];
#pragma unroll
    for (int s = 0; s < ST_MAX_STREAMS; ++s) old[s] = s < S ? xr[(size_t)s * width + c] : 0.f;
    const float yv = y[(size_t)t * ldy + c];
    float u = 0.f;
#pragma unroll
    for (int r = 0; r < ST_MAX_STREAMS; ++r) {
      if (r >= S) break;
      float v = 0.f;
#pragma unroll
      for (int s = 0; s < ST_MAX_STREAMS; ++s)
        if (s < S) v = fmaf(m[s * S + r], old[s], v);  // mix is indexed [from, to]
      v = fmaf(ow[r], yv, v);
      xr[(size_t)r * width + c] = v;
      u = fmaf(ni[r], v, u);
    }
    if (next_in) stf(out + (size_t)t * ldo, c, dyn_tanh(u, a, w[c], b[c]));
  }
}

extern "C" int jllm_streams_write(float* x, const float* y, int ldy, int n, int width, int S, const float* mix, const float* outw,
                                  const float* next_in, const float* w, const float* b, const float* alpha, void* out,
                                  int out_dtype, int ldo, hipStream_t stream) {
  if (n <= 0) return 0;
  if (width <= 0 || S < 1 || S > ST_MAX_STREAMS || ldy < width) JLLM_FAIL("streams_write: width %d, %d streams (1..%d are taken)", width, S, ST_MAX_STREAMS);
  if (!mix || !outw) JLLM_FAIL("streams_write: the mixing matrix and the output weights are needed");
  if (next_in && (!w || !b || !alpha || !out || ldo < width)) JLLM_FAIL("streams_write: the next read needs its norm and a place for its rows");
  JLLM_DISPATCH_1(out_dtype, TO, {
    streams_write_kernel<TO><<<n, ST_THREADS, 0, stream>>>(x, y, ldy, width, S, mix, outw, next_in, w, b, alpha, (TO*)out, ldo);
  })
  JLLM_CHECK_LAUNCH("streams_write");
  return 0;
}

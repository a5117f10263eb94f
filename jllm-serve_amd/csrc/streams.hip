// Several residual streams per row (hyper-connections), a norm without statistics (Dynamic Tanh), and a table row added
// by index. Everything here is element by element in fp32: no sums over a row, so a row's result depends on nothing
// but the row. The streams of a row lie side by side, x [rows, S, width] fp32.
//
//   gather_add     x[t, :] += table[ids[t], :]                        (a learned position table at the input)
//   dyntanh_read   u[c] = sum_s in[s] x[t', s, c] (in == null: the row itself, S = 1; t' = rows ? rows[t] : t);
//                  out[t, k, c] = tanh(alpha u[c]) w[c] + b[c] for k < copies, in the output's type (a sublayer's input
//                  read from the streams; the embedding's norm written once per stream; the final norm of the
//                  streams' sum over the wanted rows)
//   streams_write  every stream rewritten from the row's previous streams together: new[r] = sum_s mix[s, r] old[s] + outw[r] y, in place; and,
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

// A thread owns V neighbouring channels of one row (V = 4 where the width allows 16-byte accesses, else 1) and nothing
// else: every load it needs is requested before the first use, and no loop stands between a load and the next.
template <int V>
struct Vec;
template <>
struct Vec<1> {
  float v[1];
  __device__ __forceinline__ void load(const float* p) { v[0] = p[0]; }
  __device__ __forceinline__ void store(float* p) const { p[0] = v[0]; }
};
template <>
struct Vec<4> {
  float v[4];
  __device__ __forceinline__ void load(const float* p) {
    const float4 t = *(const float4*)p;
    v[0] = t.x, v[1] = t.y, v[2] = t.z, v[3] = t.w;
  }
  __device__ __forceinline__ void store(float* p) const { *(float4*)p = float4{v[0], v[1], v[2], v[3]}; }
};

template <int V>
__device__ __forceinline__ void store_out(float* p, const float* v) {
#pragma unroll
  for (int i = 0; i < V; ++i) p[i] = v[i];
}
template <int V>
__device__ __forceinline__ void store_out(bf16_t* p, const float* v) {
  if (V == 4) {
    uint2 t;
    t.x = (uint32_t)f32_to_bf16(v[0]).bits | ((uint32_t)f32_to_bf16(v[1]).bits << 16);
    t.y = (uint32_t)f32_to_bf16(v[2]).bits | ((uint32_t)f32_to_bf16(v[3]).bits << 16);
    *(uint2*)p = t;
  } else {
    p[0] = f32_to_bf16(v[0]);
  }
}

template <typename TO, int V, int S>
__global__ __launch_bounds__(ST_THREADS) void dyntanh_read_kernel(const float* __restrict__ x, const int* __restrict__ rows,
                                                                  int width, int streams, const float* __restrict__ in_w,
                                                                  const float* __restrict__ w, const float* __restrict__ b,
                                                                  const float* __restrict__ alpha, TO* __restrict__ out, int ldo,
                                                                  int copies) {
  const int t = blockIdx.x;
  const int c = (blockIdx.y * ST_THREADS + threadIdx.x) * V;
  if (c >= width) return;
  const float* xr = x + (size_t)(rows ? rows[t] : t) * streams * width + c;
  Vec<V> xs[S], wv, bv;
#pragma unroll
  for (int s = 0; s < S; ++s)
    if (s < streams) xs[s].load(xr + (size_t)s * width);
  wv.load(w + c);
  bv.load(b + c);
  const float a = alpha[0];
  float iw[S];
#pragma unroll
  for (int s = 0; s < S; ++s) iw[s] = (in_w && s < streams) ? in_w[s] : 1.0f;
  float o[V];
#pragma unroll
  for (int i = 0; i < V; ++i) {
    float u;
    if (in_w) {
      u = 0.f;
#pragma unroll
      for (int s = 0; s < S; ++s)
        if (s < streams) u = fmaf(iw[s], xs[s].v[i], u);
    } else {
      u = xs[0].v[i];
    }
    o[i] = dyn_tanh(u, a, wv.v[i], bv.v[i]);
  }
  for (int k = 0; k < copies; ++k) store_out<V>(out + (size_t)t * ldo + (size_t)k * width + c, o);
}

extern "C" int jllm_dyntanh_read(const float* x, const int* rows, int n, int width, int S, const float* in_w, const float* w,
                                 const float* b, const float* alpha, void* out, int out_dtype, int ldo, int copies,
                                 hipStream_t stream) {
  if (n <= 0) return 0;
  if (width <= 0 || S < 1 || S > ST_MAX_STREAMS || copies < 1 || ldo < copies * width)
    JLLM_FAIL("dyntanh_read: width %d, %d streams (1..%d are taken), %d copies in rows of %d", width, S, ST_MAX_STREAMS, copies, ldo);
  if (!in_w && S != 1) JLLM_FAIL("dyntanh_read: %d streams need their weights", S);
  if (!w || !b || !alpha) JLLM_FAIL("dyntanh_read: the norm has a weight, a bias and a slope");
  const bool vec = width % 4 == 0 && ldo % 4 == 0 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)out & 7) == 0 &&
                   ((uintptr_t)w & 15) == 0 && ((uintptr_t)b & 15) == 0;
  const int per = vec ? 4 : 1;
  dim3 grid(n, (width + ST_THREADS * per - 1) / (ST_THREADS * per));
#define ST_READ(V, SS) dyntanh_read_kernel<TO, V, SS><<<grid, ST_THREADS, 0, stream>>>(x, rows, width, S, in_w, w, b, alpha, (TO*)out, ldo, copies)
  JLLM_DISPATCH_1(out_dtype, TO, {
    if (vec && S <= 4) ST_READ(4, 4);
    else if (vec) ST_READ(4, ST_MAX_STREAMS);
    else if (S <= 4) ST_READ(1, 4);
    else ST_READ(1, ST_MAX_STREAMS);
  })
#undef ST_READ
  JLLM_CHECK_LAUNCH("dyntanh_read");
  return 0;
}

// ---------------------------------------------------------------------------------------------------------------------

template <typename TO, int V, int S>
__global__ __launch_bounds__(ST_THREADS) void streams_write_kernel(float* __restrict__ x, const float* __restrict__ y, int ldy,
                                                                   int width, int streams, const float* __restrict__ mix,
                                                                   const float* __restrict__ outw,
                                                                   const float* __restrict__ next_in, const float* __restrict__ w,
                                                                   const float* __restrict__ b, const float* __restrict__ alpha,
                                                                   TO* __restrict__ out, int ldo) {
  const int t = blockIdx.x;
  const int c = (blockIdx.y * ST_THREADS + threadIdx.x) * V;
  if (c >= width) return;
  float* xr = x + (size_t)t * streams * width + c;
  Vec<V> old[S], yv, wv, bv;
#pragma unroll
  for (int s = 0; s < S; ++s)
    if (s < streams) old[s].load(xr + (size_t)s * width);
  yv.load(y + (size_t)t * ldy + c);
  if (next_in) {
    wv.load(w + c);
    bv.load(b + c);
  }
  const float a = next_in ? alpha[0] : 0.f;
  float u[V];
#pragma unroll
  for (int i = 0; i < V; ++i) u[i] = 0.f;
#pragma unroll
  for (int r = 0; r < S; ++r) {
    if (r >= streams) break;
    const float ow = outw[r];                        // (uniform loads: the few weights of the streams)
    const float ni = next_in ? next_in[r] : 0.f;
    Vec<V> nv;
#pragma unroll
    for (int i = 0; i < V; ++i) nv.v[i] = 0.f;
#pragma unroll
    for (int s = 0; s < S; ++s) {
      if (s >= streams) break;
      const float m = mix[s * streams + r];  // row: the stream read, column: the stream written
#pragma unroll
      for (int i = 0; i < V; ++i) nv.v[i] = fmaf(m, old[s].v[i], nv.v[i]);
    }
#pragma unroll
    for (int i = 0; i < V; ++i) {
      nv.v[i] = fmaf(ow, yv.v[i], nv.v[i]);
      u[i] = fmaf(ni, nv.v[i], u[i]);
    }
    nv.store(xr + (size_t)r * width);
  }
  if (next_in) {
    float o[V];
#pragma unroll
    for (int i = 0; i < V; ++i) o[i] = dyn_tanh(u[i], a, wv.v[i], bv.v[i]);
    store_out<V>(out + (size_t)t * ldo + c, o);
  }
}

extern "C" int jllm_streams_write(float* x, const float* y, int ldy, int n, int width, int S, const float* mix, const float* outw,
                                  const float* next_in, const float* w, const float* b, const float* alpha, void* out,
                                  int out_dtype, int ldo, hipStream_t stream) {
  if (n <= 0) return 0;
  if (width <= 0 || S < 1 || S > ST_MAX_STREAMS || ldy < width) JLLM_FAIL("streams_write: width %d, %d streams (1..%d are taken)", width, S, ST_MAX_STREAMS);
  if (!mix || !outw) JLLM_FAIL("streams_write: the mixing matrix and the output weights are needed");
  if (next_in && (!w || !b || !alpha || !out || ldo < width)) JLLM_FAIL("streams_write: the next read needs its norm and a place for its rows");
  const bool vec = width % 4 == 0 && ldy % 4 == 0 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)y & 15) == 0 &&
                   (!next_in || (ldo % 4 == 0 && ((uintptr_t)out & 7) == 0 && ((uintptr_t)w & 15) == 0 && ((uintptr_t)b & 15) == 0));
  const int per = vec ? 4 : 1;
  dim3 grid(n, (width + ST_THREADS * per - 1) / (ST_THREADS * per));
#define ST_WRITE(V, SS) \
  streams_write_kernel<TO, V, SS><<<grid, ST_THREADS, 0, stream>>>(x, y, ldy, width, S, mix, outw, next_in, w, b, alpha, (TO*)out, ldo)
  JLLM_DISPATCH_1(out_dtype, TO, {
    if (vec && S <= 4) ST_WRITE(4, 4);
    else if (vec) ST_WRITE(4, ST_MAX_STREAMS);
    else if (S <= 4) ST_WRITE(1, 4);
    else ST_WRITE(1, ST_MAX_STREAMS);
  })
#undef ST_WRITE
  JLLM_CHECK_LAUNCH("streams_write");
  return 0;
}

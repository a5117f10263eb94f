// A mixture of experts whose routing is a table: row t's experts are table[token[t]][0 .. top) (a table by token id),
// or table[t][0 .. top) where a router chose them for this step's rows (`tokens` null). Everything happens on the
// device, so a step needs no answer from the GPU before it launches (and can be captured).
//
//   moe_router    one wave per row, from the router's fp32 logits z [T, E]: s = sigmoid(z) (or softmax(z) over all
//                 experts); choice = s + correction; the experts form `groups` equal groups of neighbours, a group's
//                 score is the sum of its two largest choice scores (or the largest) and only the `keep` best groups
//                 can be chosen from; the `top` largest choice scores among those win (the lowest index among equals);
//                 weights = s of the chosen / (their sum + 1e-20) * scale (or s * scale, not normalised). Writes the
//                 chosen experts [T, top] (int32) and their weights [T, top] (fp32)
//   moe_route     one workgroup: counts the assignments (row, k) of every expert, lays them out expert by expert in
//                 `sorted`, and cuts each expert's run into tiles of at most `tile_rows` rows: tiles[i] = (expert,
//                 first place in `sorted`, rows); the tiles no expert needs have 0 rows
//   moe_gemm      a grouped product over those tiles: every tile multiplies its rows with its expert's weights
//                 [N, K]. The first product gathers its input rows by token (assignment / top), applies the gate
//                 function to the two sums and writes hidden rows in the order of `sorted`; the second reads those
//                 and writes fp32 rows by assignment, or, with top = 1, adds them straight into the residual rows
//   moe_combine   residual[t] += weight * sum_k y[t * top + k], k ascending (or y[place_of[t * top + k]] where the second
//                 product wrote its rows in the order of `sorted`); with `weights` [T, top] every term has its own
//                 factor weights[t, k] as well; a shared expert's fp32 rows may join the sum, times the sigmoid of a
//                 gate logit per row
//
// The order of `sorted` within an expert comes from LDS atomics and may differ between runs; no result depends on it
// (every output is one accumulator over ascending k of its own row and weight row). This file is the fp32 path
// (plain FMAs) and takes any sizes and fp32 or bf16 operands.
#include "common.h"

#define MOE_ROUTE_THREADS 1024

__global__ __launch_bounds__(MOE_ROUTE_THREADS) void moe_route_kernel(const int* __restrict__ tokens, const int* __restrict__ table,
                                                                     int T, int top, int E, int tile_rows, int max_tiles,
                                                                     int* __restrict__ sorted, int* __restrict__ tiles,
                                                                     int* __restrict__ place_of) {
  extern __shared__ int sh[];
  int* count = sh;           // [E]
  int* start = sh + E;       // [E + 1]
  int* tile0 = sh + 2 * E + 1;  // [E + 1]
  int* cursor = sh + 3 * E + 2;  // [E]
  const int A = T * top;
  for (int e = threadIdx.x; e < E; e += MOE_ROUTE_THREADS) count[e] = 0, cursor[e] = 0;
  for (int i = threadIdx.x; i < max_tiles; i += MOE_ROUTE_THREADS) {
    tiles[3 * i] = 0;
    tiles[3 * i + 1] = 0;
    tiles[3 * i + 2] = 0;
  }
  __syncthreads();
  for (int a = threadIdx.x; a < A; a += MOE_ROUTE_THREADS) {
    const int e = table[(size_t)(tokens ? tokens[a / top] : a / top) * top + a % top];
    atomicAdd(&count[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int s = 0, t = 0;
    for (int e = 0; e < E; ++e) {
      start[e] = s;
      tile0[e] = t;
      s += count[e];
      t += (count[e] + tile_rows - 1) / tile_rows;
    }
    start[E] = s;
    tile0[E] = t;
  }
  __syncthreads();
  for (int a = threadIdx.x; a < A; a += MOE_ROUTE_THREADS) {
    const int e = table[(size_t)(tokens ? tokens[a / top] : a / top) * top + a % top];
    const int place = start[e] + atomicAdd(&cursor[e], 1);
    sorted[place] = a;
    if (place_of) place_of[a] = place;
  }
  for (int e = threadIdx.x; e < E; e += MOE_ROUTE_THREADS) {
    const int c = count[e];
    for (int k = 0; k * tile_rows < c; ++k) {
      const int i = tile0[e] + k;
      if (i >= max_tiles) break;
      tiles[3 * i] = e;
      tiles[3 * i + 1] = start[e] + k * tile_rows;
      tiles[3 * i + 2] = min(tile_rows, c - k * tile_rows);
    }
  }
}

extern "C" int jllm_moe_route(const int* tokens, const int* table, int T, int top, int E, int tile_rows, int max_tiles,
                              int* sorted, int* tiles, int* place_of, hipStream_t stream) {
  if (T <= 0) return 0;
  if (top <= 0 || E <= 0 || top > E || tile_rows <= 0) JLLM_FAIL("moe_route: top %d of %d experts, tiles of %d rows", top, E, tile_rows);
  const long A = (long)T * top;
  const long need = A / tile_rows + E < A ? A / tile_rows + E : A;
  if (max_tiles < need) JLLM_FAIL("moe_route: room for %d tiles, %ld may be needed", max_tiles, need);
  const size_t smem = (size_t)(4 * E + 2) * sizeof(int);
  if (smem > 64 * 1024) JLLM_FAIL("moe_route: %d experts are more than this kernel's LDS holds", E);
  moe_route_kernel<<<1, MOE_ROUTE_THREADS, smem, stream>>>(tokens, table, T, top, E, tile_rows, max_tiles, sorted, tiles, place_of);
  JLLM_CHECK_LAUNCH("moe_route");
  return 0;
}

// ---------------------------------------------------------------------------------------------------------------
#define MG_ROWS 16
#define MG_COLS 64
#define MG_K 32

// in_map 0: input row = place in `sorted`; 1: the assignment's token row (sorted[place] / top).
// out_map 0: output row = place in `sorted`; 1: the assignment (sorted[place]); 2: add weight * v into the fp32 row of
// the assignment's token (top = 1 only: no two assignments share a row).
template <typename TA, typename TW, bool GATED>
__global__ __launch_bounds__(256) void moe_gemm_generic_kernel(
    const TA* __restrict__ A, int lda, const TW* __restrict__ W, const TW* __restrict__ W2, void* __restrict__ out,
    int out_dtype, int ldo, int N, int K, const int* __restrict__ sorted, const int* __restrict__ tiles, int top,
    int in_map, int out_map, float weight, GateSpec gs) {
  const int tile = blockIdx.y;
  // a tile of more than MG_ROWS rows is taken MG_ROWS at a time, over gridDim.z
  const int rows = min(MG_ROWS, tiles[3 * tile + 2] - MG_ROWS * (int)blockIdx.z);
  if (rows <= 0) return;
  const int e = tiles[3 * tile], first = tiles[3 * tile + 1] + MG_ROWS * (int)blockIdx.z;
  __shared__ float As[MG_K][MG_ROWS + 1];
  __shared__ float Ws[MG_K][MG_COLS + 4];
  __shared__ float Us[GATED ? MG_K : 1][MG_COLS + 4];
  __shared__ int src[MG_ROWS], asg[MG_ROWS];
  if (threadIdx.x < MG_ROWS) {
    const int place = first + min((int)threadIdx.x, rows - 1);
    const int a = sorted[place];
    asg[threadIdx.x] = a;
    src[threadIdx.x] = in_map ? a / top : place;
  }
  __syncthreads();
  const int n0 = blockIdx.x * MG_COLS;
  const TW* w = W + (size_t)e * N * K;
  const TW* w2 = GATED ? W2 + (size_t)e * N * K : nullptr;
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  float acc[4] = {}, acc2[4] = {};
  for (int k0 = 0; k0 < K; k0 += MG_K) {
    for (int i = threadIdx.x; i < MG_ROWS * MG_K; i += 256) {
      const int r = i / MG_K, k = i % MG_K;
      As[k][r] = (r < rows && k0 + k < K) ? ldf(A + (size_t)src[r] * lda, k0 + k) : 0.f;
    }
    for (int i = threadIdx.x; i < MG_COLS * MG_K; i += 256) {
      const int r = i / MG_K, k = i % MG_K;
      const bool in = n0 + r < N && k0 + k < K;
      Ws[k][r] = in ? ldf(w + (size_t)(n0 + r) * K, k0 + k) : 0.f;
      if (GATED) Us[k][r] = in ? ldf(w2 + (size_t)(n0 + r) * K, k0 + k) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < MG_K; ++kk) {
      const float av = As[kk][ty];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        acc[j] = fmaf(av, Ws[kk][tx * 4 + j], acc[j]);
        if (GATED) acc2[j] = fmaf(av, Us[kk][tx * 4 + j], acc2[j]);
      }
    }
    __syncthreads();
  }
  if (ty >= rows) return;
  const size_t orow = out_map == 0 ? (size_t)(first + ty) : out_map == 1 ? (size_t)asg[ty] : (size_t)(asg[ty] / top);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int n = n0 + tx * 4 + j;
    if (n >= N) continue;
    float v = acc[j];
    if (GATED) v = gated<false>(v, acc2[j], gs);
    const size_t o = orow * ldo + n;
    if (out_map == 2)
      ((float*)out)[o] += weight * v;
    else if (out_dtype == JLLM_BF16)
      stf((bf16_t*)out, o, v);
    else
      stf((float*)out, o, v);
  }
}

extern "C" int jllm_moe_gemm_generic(const void* A, int a_dtype, int lda, const void* W, const void* W2, int w_dtype,
                                     void* out, int out_dtype, int ldo, int N, int K, const int* sorted, const int* tiles,
                                     int max_tiles, int tile_rows, int top, int in_map, int out_map, float weight,
                                     int epilogue, float gate_limit, hipStream_t stream) {
  if (max_tiles <= 0) return 0;
  if (N <= 0 || K <= 0 || lda < K || ldo < N) JLLM_FAIL("moe_gemm: N %d K %d lda %d ldo %d", N, K, lda, ldo);
  if (tile_rows <= 0 || tile_rows % MG_ROWS) JLLM_FAIL("moe_gemm: this kernel takes tiles of multiples of %d rows, the route made %d", MG_ROWS, tile_rows);
  if (max_tiles > 65535) JLLM_FAIL("moe_gemm: %d tiles are too many for one launch", max_tiles);
  JLLM_TAKE_GATE("moe_gemm", epilogue, gate_limit, gs);
  if ((epilogue != 0 && epilogue != 2) || (epilogue == 2) != (W2 != nullptr)) JLLM_FAIL("moe_gemm: epilogue %d", epilogue);
  if (in_map < 0 || in_map > 1 || out_map < 0 || out_map > 2) JLLM_FAIL("moe_gemm: maps %d / %d", in_map, out_map);
  if (out_map == 2 && (top != 1 || out_dtype != JLLM_F32)) JLLM_FAIL("moe_gemm: adding into the token's row needs top = 1 and fp32 rows");
  dim3 grid((N + MG_COLS - 1) / MG_COLS, max_tiles, tile_rows / MG_ROWS);
  JLLM_DISPATCH_1(a_dtype, TA, {
    JLLM_DISPATCH_1(w_dtype, TW, {
      if (W2)
        moe_gemm_generic_kernel<TA, TW, true><<<grid, 256, 0, stream>>>((const TA*)A, lda, (const TW*)W, (const TW*)W2, out, out_dtype,
                                                                        ldo, N, K, sorted, tiles, top, in_map, out_map, weight, gs);
      else
        moe_gemm_generic_kernel<TA, TW, false><<<grid, 256, 0, stream>>>((const TA*)A, lda, (const TW*)W, nullptr, out, out_dtype, ldo,
                                                                         N, K, sorted, tiles, top, in_map, out_map, weight, gs);
    })
  })
  JLLM_CHECK_LAUNCH("moe_gemm_generic");
  return 0;
}

// ---------------------------------------------------------------------------------------------------------------
// A thread owns V neighbouring channels of one row (V = 4 where the width allows 16-byte accesses, else 1): the places
// and weights of the row's `top` terms, the residual and the shared row are requested before the sum starts, and the
// terms' loads do not wait for one another. Every output is still one chain of multiply-adds over ascending k.
template <int V>
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ y, float* __restrict__ residual, int width,
                                                         int top, float weight, const int* __restrict__ place_of,
                                                         const float* __restrict__ weights, const float* __restrict__ shared,
                                                         const float* __restrict__ shared_gate, int ldsg, int overwrite,
                                                         int ld_shared) {
  const int t = blockIdx.x;
  const int i = (blockIdx.y * 256 + threadIdx.x) * V;
  if (i >= width) return;
  // a shared expert's rows join the sum, times sigmoid of the row's gate logit where it has one
  const float sg = shared ? (shared_gate ? 1.0f / (1.0f + expf(-shared_gate[(size_t)t * ldsg])) : 1.0f) : 0.f;
  float r[V], sh[V], s[V];
#pragma unroll
  for (int c = 0; c < V; ++c) {
    r[c] = overwrite ? 0.f : residual[(size_t)t * width + i + c];
    sh[c] = shared ? shared[(size_t)t * ld_shared + i + c] : 0.f;
    s[c] = 0.f;
  }
#pragma unroll 4
  for (int k = 0; k < top; ++k) {
    const size_t row = place_of ? (size_t)place_of[t * top + k] : (size_t)t * top + k;
    const float w = weights ? weights[(size_t)t * top + k] : 1.0f;
    float v[V];
    if (V == 4) {
      const float4 q = *(const float4*)(y + row * width + i);
      v[0] = q.x, v[1 % V] = q.y, v[2 % V] = q.z, v[3 % V] = q.w;
    } else {
      v[0] = y[row * width + i];
    }
#pragma unroll
    for (int c = 0; c < V; ++c) s[c] = weights ? fmaf(w, v[c], s[c]) : s[c] + v[c];
  }
#pragma unroll
  for (int c = 0; c < V; ++c) {
    float o = r[c];
    if (shared) o = fmaf(sg, sh[c], o);
    residual[(size_t)t * width + i + c] = o + weight * s[c];
  }
}

// `shared` [T, width] fp32, rows `ld_shared` apart (optional): one more term per row, times sigmoid(shared_gate[t * ldsg]) where a gate is given;
// `overwrite`: the rows of `residual` are written, not added to (it may be the same tensor as `shared`)
extern "C" int jllm_moe_combine(const float* y, float* residual, int T, int width, int top, float weight, const int* place_of,
                                const float* weights, const float* shared, const float* shared_gate, int ldsg, int overwrite,
                                int ld_shared, hipStream_t stream) {
  if (T <= 0) return 0;
  if (width <= 0 || top <= 0) JLLM_FAIL("moe_combine: width %d top %d", width, top);
  if (shared_gate && !shared) JLLM_FAIL("moe_combine: a gate without the shared rows it weighs");
  if (shared && ld_shared < width) JLLM_FAIL("moe_combine: shared rows %d apart for a width of %d", ld_shared, width);
  const bool vec = width % 4 == 0 && ((uintptr_t)y & 15) == 0;
  const int per = vec ? 4 : 1;
  dim3 grid(T, (width + 256 * per - 1) / (256 * per));
  if (vec)
    moe_combine_kernel<4><<<grid, 256, 0, stream>>>(y, residual, width, top, weight, place_of, weights, shared, shared_gate, ldsg,
                                                    overwrite, ld_shared);
  else
    moe_combine_kernel<1><<<grid, 256, 0, stream>>>(y, residual, width, top, weight, place_of, weights, shared, shared_gate, ldsg,
                                                    overwrite, ld_shared);
  JLLM_CHECK_LAUNCH("moe_combine");
  return 0;
}

// ---------------------------------------------------------------------------------------------------------------
// LDS: s [E] | choice [E] | group score [groups] | group allowed [groups]
template <typename TC>
__global__ __launch_bounds__(64) void moe_router_kernel(const float* __restrict__ z, int ldz, const TC* __restrict__ correction,
                                                       int E, int groups, int keep, int top, float scale,
                                                       int* __restrict__ chosen, float* __restrict__ weights, int softmax,
                                                       int group_max, int normalize) {
  extern __shared__ float rs[];
  float* s = rs;
  float* choice = rs + E;
  float* gscore = rs + 2 * E;
  int* allowed = (int*)(rs + 2 * E + groups);
  const int t = blockIdx.x, lane = threadIdx.x;
  const int per = E / groups;
  float zmax = -INFINITY, zden = 1.0f;
  if (softmax) {  // s = softmax(z) over all experts
    for (int e = lane; e < E; e += 64) zmax = fmaxf(zmax, z[(size_t)t * ldz + e]);
    zmax = wave_max(zmax);
    float d = 0.f;
    for (int e = lane; e < E; e += 64) d += expf(z[(size_t)t * ldz + e] - zmax);
    zden = wave_sum(d);
  }
  for (int e = lane; e < E; e += 64) {
    const float v = softmax ? expf(z[(size_t)t * ldz + e] - zmax) / zden : 1.0f / (1.0f + expf(-z[(size_t)t * ldz + e]));
    s[e] = v;
    choice[e] = v + (correction ? ldf(correction, e) : 0.f);
  }
  __syncthreads();
  for (int g = lane; g < groups; g += 64) {  // the sum of the group's two largest choice scores
    float a = -INFINITY, b = -INFINITY;
    for (int i = 0; i < per; ++i) {
      const float v = choice[g * per + i];
      if (v > a) b = a, a = v; else if (v > b) b = v;
    }
    gscore[g] = (per > 1 && !group_max) ? a + b : a;
    allowed[g] = 0;
  }
  __syncthreads();
  if (lane == 0) {
    for (int n = 0; n < keep; ++n) {
      int best = -1;
      for (int g = 0; g < groups; ++g)
        if (!allowed[g] && (best < 0 || gscore[g] > gscore[best])) best = g;
      if (best >= 0) allowed[best] = 1;
    }
  }
  __syncthreads();
  for (int e = lane; e < E; e += 64)
    if (!allowed[e / per]) choice[e] = -INFINITY;
  __syncthreads();
  float sum = 0.f;
  for (int k = 0; k < top; ++k) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {  // ascending e: the lowest index among equals stays
      const float v = choice[e];
      if (v > bv) bv = v, bi = e;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ov > bv || (ov == bv && oi < bi)) bv = ov, bi = oi;
    }
    if (bi >= E) bi = 0;  // nothing left to choose from: the entry point refuses the configurations where this could be
    const float sv = s[bi];
    sum += sv;
    if (lane == 0) {
      chosen[(size_t)t * top + k] = bi;
      weights[(size_t)t * top + k] = sv;  // the raw score; scaled below once the sum is known
      choice[bi] = -INFINITY;
    }
    __syncthreads();
  }
  if (lane == 0)
    for (int k = 0; k < top; ++k)
      weights[(size_t)t * top + k] = normalize ? weights[(size_t)t * top + k] / (sum + 1e-20f) * scale : weights[(size_t)t * top + k] * scale;
}

extern "C" int jllm_moe_router(const float* z, int ldz, const void* correction, int c_dtype, int T, int E, int groups, int keep,
                               int top, float scale, int* chosen, float* weights, int softmax, int group_max, int normalize,
                               hipStream_t stream) {
  if (T <= 0) return 0;
  if (E <= 0 || top <= 0 || top > E || ldz < E) JLLM_FAIL("moe_router: top %d of %d experts in rows of %d", top, E, ldz);
  if (groups <= 0 || E % groups || keep <= 0 || keep > groups || keep * (E / groups) < top)
    JLLM_FAIL("moe_router: %d experts in %d groups of which %d are kept, for top %d", E, groups, keep, top);
  const size_t smem = (size_t)(2 * E + 2 * groups) * sizeof(float);
  if (smem > 64 * 1024) JLLM_FAIL("moe_router: %d experts are more than this kernel's LDS holds", E);
  JLLM_DISPATCH_1(c_dtype, TC, {
    moe_router_kernel<TC><<<T, 64, smem, stream>>>(z, ldz, (const TC*)correction, E, groups, keep, top, scale, chosen, weights, softmax,
                                                   group_max, normalize);
  })
  JLLM_CHECK_LAUNCH("moe_router");
  return 0;
}

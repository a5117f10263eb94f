// Latent attention for any sizes, fp32 or bf16 storage, all arithmetic in fp32 with plain FMAs: the 32-bit path of
// the mixer and the fallback for shapes the matrix-core kernels refuse.
//
// A layer caches per position one row of Dk = R + Dr numbers: the RMS-normed latent c (R) and a rotated key part
// (Dr) that all heads share. Head h's unrotated key is W_uk[h] c and its value W_uv[h] c, so with
// qa[h] = [W_uk[h]^T q_plain[h] | q_rot[h]] the score of a key is qa[h] . row, and the head's output is
// W_uv[h] (sum_j p_j c_j): every head attends over the same rows (their first R entries are the values), and the two
// per-head products sit before and after the attention. Three kernels here:
//
//   latent_prepare      per row of the down-projections' output: RMSNorm of the query latent (written out), RMSNorm
//                       of c and rotation of the key part at the row's position (both stored at the row's cache slot)
//   latent_heads        out[t, h, :] = W[h] in[t, h, :] for all heads in one launch (W[h] is [N, K] row-major), with
//                       a tail per head that is rotated and copied (the query side), or the result multiplied by
//                       sigmoid of a gate row (the value side)
//   latent_attention    paged causal attention of qa over the rows with a window and a per-head sink in the softmax's
//                       denominator; key blocks of 64 aligned to absolute positions, four waves over alternating
//                       blocks merged in wave order, so a row's result depends on its own position and keys only
//
// Rotation ("half" pairing): dimension i < dims/2 of the rotated part is paired with i + dims/2:
// (u, v) -> (u cos a - v sin a, v cos a + u sin a), cos and sin from the position's row of the fp32 tables;
// entries from `dims` on pass unchanged.
#include <math.h>

#include "common.h"

// ---------------------------------------------------------------------------------------------------------------
template <typename T, typename TG>
__global__ __launch_bounds__(256) void latent_prepare_kernel(
    const T* __restrict__ y, int ldy, int q_off, int q_rank, int kv_off, int R, int Dr, int rot_dims,
    const TG* __restrict__ gq, const TG* __restrict__ gkv, float eps, const int* __restrict__ positions,
    const int* __restrict__ slots, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    T* __restrict__ cq, int ldcq, T* __restrict__ cache) {
  __shared__ float red[4];
  const int t = blockIdx.x;
  const T* row = y + (size_t)t * ldy;
  if (q_rank > 0) {  // a mixer without a query latent has nothing to norm here
    float ss = 0.f;
    for (int i = threadIdx.x; i < q_rank; i += 256) {
      const float v = ldf(row, q_off + i);
      ss = fmaf(v, v, ss);
    }
    ss = block_sum<4>(ss, red);
    const float s = norm_scale(ss, q_rank, eps);
    for (int i = threadIdx.x; i < q_rank; i += 256) stf(cq + (size_t)t * ldcq, i, (ldf(row, q_off + i) * s) * ldf(gq, i));
  }
  if (!cache) return;
  const int slot = slots[t];
  if (slot < 0) return;  // a padding row of a captured step: stores nothing
  T* dst = cache + (size_t)slot * (R + Dr);
  float ss = 0.f;
  for (int i = threadIdx.x; i < R; i += 256) {
    const float v = ldf(row, kv_off + i);
    ss = fmaf(v, v, ss);
  }
  ss = block_sum<4>(ss, red);
  const float s = norm_scale(ss, R, eps);
  for (int i = threadIdx.x; i < R; i += 256) stf(dst, i, (ldf(row, kv_off + i) * s) * ldf(gkv, i));
  const int half = rot_dims >> 1;
  const size_t at = (size_t)positions[t] * half;
  const T* kr = row + kv_off + R;
  for (int i = threadIdx.x; i < Dr; i += 256) {
    float v = ldf(kr, i);
    if (i < half) {
      v = v * cos_t[at + i] - ldf(kr, i + half) * sin_t[at + i];
    } else if (i < rot_dims) {
      v = v * cos_t[at + i - half] + ldf(kr, i - half) * sin_t[at + i - half];
    }
    stf(dst, R + i, v);
  }
}

extern "C" int jllm_latent_prepare(const void* y, int dtype, int ldy, int n_rows, int q_off, int q_rank, int kv_off,
                                   int R, int Dr, int rot_dims, const void* gq, const void* gkv, int gain_dtype,
                                   float eps, const int* positions, const int* slots, const float* cos_t,
                                   const float* sin_t, void* cq, int ldcq, void* cache, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (q_rank == 0 && !cache) return 0;
  if (q_rank < 0 || (q_rank > 0 && !cq) || ldcq < q_rank || q_off < 0 || q_off + q_rank > ldy) JLLM_FAIL("latent_prepare: query latent of %d at %d in rows of %d", q_rank, q_off, ldy);
  if (cache) {
    if (R <= 0 || Dr < 0 || kv_off < 0 || kv_off + R + Dr > ldy) JLLM_FAIL("latent_prepare: latent of %d + %d at %d in rows of %d", R, Dr, kv_off, ldy);
    if (rot_dims < 0 || rot_dims > Dr || (rot_dims & 1)) JLLM_FAIL("latent_prepare: %d rotated dims of %d", rot_dims, Dr);
    if (!slots || !positions || (rot_dims && (!cos_t || !sin_t))) JLLM_FAIL("latent_prepare: a cache store needs slots, positions and the rotation's tables");
  }
  JLLM_DISPATCH_1(dtype, T, {
    JLLM_DISPATCH_1(gain_dtype, TG, {
      latent_prepare_kernel<T, TG><<<n_rows, 256, 0, stream>>>((const T*)y, ldy, q_off, q_rank, kv_off, R, Dr, rot_dims,
                                                             (const TG*)gq, (const TG*)gkv, eps, positions, slots, cos_t,
                                                             sin_t, (T*)cq, ldcq, (T*)cache);
    })
  })
  JLLM_CHECK_LAUNCH("latent_prepare");
  return 0;
}

// ---------------------------------------------------------------------------------------------------------------
// out[t, h, n] = sum_k W[h][n][k] * in[t, h, k], one accumulator per output in ascending k. Tiles of 64 rows by 64
// outputs of one head, K in steps of 32 through LDS. mode 0: the head's `tail` entries behind its K inputs are rotated
// at the row's position (the first rot_dims of them) and copied behind its N outputs; mode 1: every output is
// multiplied by sigmoid(gate[t, h * N + n]).
#define LH_T 64
#define LH_K 32

template <typename T, typename TW>
__global__ __launch_bounds__(256) void latent_heads_kernel(
    const T* __restrict__ in, int ld_in, int in_hstride, const TW* __restrict__ W, T* __restrict__ out, int ld_out,
    int out_hstride, int M, int N, int K, int mode, int tail, int rot_dims, const int* __restrict__ positions,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, const T* __restrict__ gate, int ld_gate) {
  __shared__ float As[LH_K][LH_T + 4];
  __shared__ float Ws[LH_K][LH_T + 4];
  const int h = blockIdx.z;
  const int m0 = blockIdx.y * LH_T;
  const int n_tiles = (N + LH_T - 1) / LH_T;
  const T* a = in + (size_t)h * in_hstride;
  T* o = out + (size_t)h * out_hstride;
  if ((int)blockIdx.x == n_tiles) {  // mode 0: the rotated tail of this head, rows m0 .. m0 + 63
    const int half = rot_dims >> 1;
    for (int e = threadIdx.x; e < LH_T * tail; e += 256) {
      const int m = m0 + e / tail, i = e % tail;
      if (m >= M) break;
      const T* src = a + (size_t)m * ld_in + K;
      const size_t at = (size_t)positions[m] * half;
      float v = ldf(src, i);
      if (i < half)
        v = v * cos_t[at + i] - ldf(src, i + half) * sin_t[at + i];
      else if (i < rot_dims)
        v = v * cos_t[at + i - half] + ldf(src, i - half) * sin_t[at + i - half];
      stf(o + (size_t)m * ld_out, N + i, v);
    }
    return;
  }
  const int n0 = blockIdx.x * LH_T;
  const TW* w = W + (size_t)h * N * K;
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += LH_K) {
    for (int e = threadIdx.x; e < LH_T * LH_K; e += 256) {
      const int r = e / LH_K, k = e % LH_K;
      As[k][r] = (m0 + r < M && k0 + k < K) ? ldf(a + (size_t)(m0 + r) * ld_in, k0 + k) : 0.f;
      Ws[k][r] = (n0 + r < N && k0 + k < K) ? ldf(w + (size_t)(n0 + r) * K, k0 + k) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < LH_K; ++kk) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = As[kk][ty * 4 + i], wv[i] = Ws[kk][tx * 4 + i];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (mode == 1) v = v / (1.0f + expf(-ldf(gate + (size_t)m * ld_gate, (size_t)h * N + n)));
      stf(o + (size_t)m * ld_out, n, v);
    }
  }
}

extern "C" int jllm_latent_heads_generic(const void* in, int dtype, int ld_in, int in_hstride, const void* W, int w_dtype,
                                         void* out, int ld_out, int out_hstride, int M, int H, int N, int K, int mode,
                                         int tail, int rot_dims, const int* positions, const float* cos_t,
                                         const float* sin_t, const void* gate, int ld_gate, hipStream_t stream) {
  if (M <= 0) return 0;
  if (H <= 0 || N <= 0 || K <= 0 || H > 65535) JLLM_FAIL("latent_heads: %d heads of %d x %d", H, N, K);
  if (mode != 0 && mode != 1) JLLM_FAIL("latent_heads: mode %d", mode);
  if (mode == 0 && (tail < 0 || rot_dims < 0 || rot_dims > tail || (rot_dims & 1))) JLLM_FAIL("latent_heads: a tail of %d with %d rotated", tail, rot_dims);
  if (mode == 0 && tail > 0 && (!positions || (rot_dims && (!cos_t || !sin_t)))) JLLM_FAIL("latent_heads: the rotated tail needs positions and tables");
  if (mode == 1 && (!gate || ld_gate < H * N)) JLLM_FAIL("latent_heads: the gated form needs a gate row of %d", H * N);
  if (ld_in < (H - 1) * in_hstride + K + (mode == 0 ? tail : 0) || ld_out < (H - 1) * out_hstride + N + (mode == 0 ? tail : 0))
    JLLM_FAIL("latent_heads: rows of %d / %d do not hold %d heads", ld_in, ld_out, H);
  const int n_tiles = (N + LH_T - 1) / LH_T;
  dim3 grid(n_tiles + ((mode == 0 && tail > 0) ? 1 : 0), (M + LH_T - 1) / LH_T, H);
  if (grid.y > 65535) JLLM_FAIL("latent_heads: %d rows are too many for one launch", M);
  JLLM_DISPATCH_1(dtype, T, {
    JLLM_DISPATCH_1(w_dtype, TW, {
      latent_heads_kernel<T, TW><<<grid, 256, 0, stream>>>((const T*)in, ld_in, in_hstride, (const TW*)W, (T*)out, ld_out,
                                                           out_hstride, M, N, K, mode, mode == 0 ? tail : 0, rot_dims,
                                                           positions, cos_t, sin_t, (const T*)gate, ld_gate);
    })
  })
  JLLM_CHECK_LAUNCH("latent_heads");
  return 0;
}

// ---------------------------------------------------------------------------------------------------------------
// One workgroup of four waves per (row, GC heads). The row at position p sees keys [first, p], first = max(0, p + 1 -
// window) with a window, else 0. Within a 64-key block a lane owns one key for the scores (ascending dims) and
// 64-strided value dims for the weighted sum (ascending keys). All heads read the same rows.
#define LA_MAX_ACC 16  // R <= 1024
#define LA_WAVES 4

template <typename T>
__device__ __forceinline__ void la_load4(const T* __restrict__ p, float (&v)[4]);
template <>
__device__ __forceinline__ void la_load4<float>(const float* __restrict__ p, float (&v)[4]) {
  const float4 t = *(const float4*)p;
  v[0] = t.x, v[1] = t.y, v[2] = t.z, v[3] = t.w;
}
template <>
__device__ __forceinline__ void la_load4<bf16_t>(const bf16_t* __restrict__ p, float (&v)[4]) {
  const uint2 t = *(const uint2*)p;
  v[0] = __builtin_bit_cast(float, t.x << 16), v[1] = __builtin_bit_cast(float, t.x & 0xffff0000u);
  v[2] = __builtin_bit_cast(float, t.y << 16), v[3] = __builtin_bit_cast(float, t.y & 0xffff0000u);
}

template <typename T, int GC>
__global__ __launch_bounds__(64 * LA_WAVES) void latent_attention_generic_kernel(
    const T* __restrict__ qa, int ldq, T* __restrict__ out, int ldo, const T* __restrict__ cache,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ row_req,
    const int* __restrict__ positions, int H, int R, int Dk, int page_size, int window, float scale,
    const float* __restrict__ sink, int wide) {
  extern __shared__ float smem[];
  float* qs = smem;            // GC x Dk
  float* mg = smem + GC * Dk;  // LA_WAVES x GC x (2 + R)
  const int t = blockIdx.x;
  const int h0 = blockIdx.y * GC;
  const int gn = min(GC, H - h0);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int pos = positions[t];
  const int* tbl = block_table + (size_t)row_req[t] * max_blocks;
  const int first = window > 0 ? max(0, pos + 1 - window) : 0;
  for (int i = threadIdx.x; i < GC * Dk; i += 64 * LA_WAVES) {
    const int g = min(i / Dk, gn - 1);
    qs[i] = ldf(qa + (size_t)t * ldq + (size_t)(h0 + g) * Dk, i % Dk);
  }
  __syncthreads();
  const int nacc = (R + 63) >> 6;
  const int dk4 = wide ? (Dk & ~3) : 0;
  float acc[GC][LA_MAX_ACC];
  float m[GC], l[GC];
#pragma unroll
  for (int g = 0; g < GC; ++g) {
    m[g] = -INFINITY, l[g] = 0.f;
#pragma unroll
    for (int a = 0; a < LA_MAX_ACC; ++a) acc[g][a] = 0.f;
  }
  const int b_first = first >> 6;
  for (int blk = b_first + ((wave - b_first) & (LA_WAVES - 1)); blk * 64 <= pos; blk += LA_WAVES) {
    const int c0 = blk * 64;
    const int kj = c0 + lane;
    const bool valid = kj >= first && kj <= pos;
    float s[GC];
#pragma unroll
    for (int g = 0; g < GC; ++g) s[g] = -INFINITY;
    size_t row_at = 0;
    if (valid) {
      const int page = tbl[kj / page_size];
      row_at = ((size_t)page * page_size + kj % page_size) * Dk;
      const T* kr = cache + row_at;
      float d[GC];
#pragma unroll
      for (int g = 0; g < GC; ++g) d[g] = 0.f;
#pragma unroll 4
      for (int i = 0; i < dk4; i += 4) {
        float kv[4];
        la_load4<T>(kr + i, kv);
#pragma unroll
        for (int g = 0; g < GC; ++g)
#pragma unroll
          for (int e = 0; e < 4; ++e) d[g] = fmaf(qs[g * Dk + i + e], kv[e], d[g]);
      }
      for (int i = dk4; i < Dk; ++i) {
        const float kv = ldf(kr, i);
#pragma unroll
        for (int g = 0; g < GC; ++g) d[g] = fmaf(qs[g * Dk + i], kv, d[g]);
      }
#pragma unroll
      for (int g = 0; g < GC; ++g) s[g] = d[g] * scale;
    }
    float p[GC];
#pragma unroll
    for (int g = 0; g < GC; ++g) {
      const float m_new = fmaxf(m[g], wave_max(s[g]));
      p[g] = valid ? expf(s[g] - m_new) : 0.f;
      const float alpha = expf(m[g] - m_new);
      l[g] = l[g] * alpha + wave_sum(p[g]);
#pragma unroll
      for (int a = 0; a < LA_MAX_ACC; ++a) acc[g][a] *= alpha;
      m[g] = m_new;
    }
    const int j0 = max(0, first - c0);
    const int j1 = min(63, pos - c0);
    for (int jb = 0; jb < 64; jb += 4) {
      if (jb + 3 < j0 || jb > j1) continue;
      float pj[4][GC], vv[4][LA_MAX_ACC];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int j = jb + u;
        const int jj = min(max(j, j0), j1);  // a key outside the range has probability 0 and reads one inside it
#pragma unroll
        for (int g = 0; g < GC; ++g) pj[u][g] = __shfl(p[g], j, 64);
        const unsigned lo = __shfl((unsigned)(row_at & 0xffffffffu), jj, 64), hi = __shfl((unsigned)(row_at >> 32), jj, 64);
        const T* vr = cache + (((size_t)hi << 32) | lo);
#pragma unroll
        for (int a = 0; a < LA_MAX_ACC; ++a) {
          const int d = lane + a * 64;
          vv[u][a] = (a < nacc && d < R) ? ldf(vr, d) : 0.f;
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int g = 0; g < GC; ++g)
#pragma unroll
          for (int a = 0; a < LA_MAX_ACC; ++a)
            if (a < nacc) acc[g][a] = fmaf(pj[u][g], vv[u][a], acc[g][a]);
    }
  }
#pragma unroll
  for (int g = 0; g < GC; ++g) {
    float* mine = mg + (size_t)(wave * GC + g) * (2 + R);
    if (lane == 0) {
      mine[0] = m[g];
      mine[1] = l[g];
    }
#pragma unroll
    for (int a = 0; a < LA_MAX_ACC; ++a) {
      const int d = lane + a * 64;
      if (a < nacc && d < R) mine[2 + d] = acc[g][a];
    }
  }
  __syncthreads();
  if (wave != 0) return;
#pragma unroll
  for (int g = 0; g < GC; ++g) {
    if (g >= gn) continue;
    float mm = m[g], ll = l[g];
    for (int w = 1; w < LA_WAVES; ++w) {
      const float* theirs = mg + (size_t)(w * GC + g) * (2 + R);
      const float om = theirs[0], ol = theirs[1];
      if (ol == 0.f) continue;  // that wave had no key
      const float m_new = fmaxf(mm, om);
      const float ca = expf(mm - m_new), cb = expf(om - m_new);
      ll = ll * ca + ol * cb;
#pragma unroll
      for (int a = 0; a < LA_MAX_ACC; ++a) {
        const int d = lane + a * 64;
        if (a < nacc && d < R) acc[g][a] = acc[g][a] * ca + theirs[2 + d] * cb;
      }
      mm = m_new;
    }
    if (sink) {  // exp(sink) joins the denominator: it has no key and no value and is not scaled
      const float sk = sink[h0 + g];
      const float m_new = fmaxf(mm, sk);
      const float ca = expf(mm - m_new);
      ll = ll * ca + expf(sk - m_new);
#pragma unroll
      for (int a = 0; a < LA_MAX_ACC; ++a) acc[g][a] *= ca;
    }
    const float inv = 1.0f / ll;
    T* o = out + (size_t)t * ldo + (size_t)(h0 + g) * R;
#pragma unroll
    for (int a = 0; a < LA_MAX_ACC; ++a) {
      const int d = lane + a * 64;
      if (a < nacc && d < R) stf(o, d, acc[g][a] * inv);
    }
  }
}

extern "C" int jllm_latent_attention_generic(const void* qa, int ldq, void* out, int ldo, int dtype, const void* cache,
                                             const int* block_table, int max_blocks, const int* row_req,
                                             const int* positions, int n_rows, int H, int R, int Dk, int page_size,
                                             int window, float scale, const float* sink, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (H <= 0 || H > 65535) JLLM_FAIL("latent attention: %d heads", H);
  if (R <= 0 || R > 64 * LA_MAX_ACC || Dk < R) JLLM_FAIL("latent attention: latent of %d in rows of %d (this kernel takes latents up to %d)", R, Dk, 64 * LA_MAX_ACC);
  if (page_size <= 0 || max_blocks <= 0) JLLM_FAIL("latent attention: page_size %d max_blocks %d", page_size, max_blocks);
  if (ldq < H * Dk || ldo < H * R) JLLM_FAIL("latent attention: row strides %d/%d", ldq, ldo);
  if (window < 0) JLLM_FAIL("latent attention: window %d", window);
  int cus = jllm_compute_units();
  if (cus <= 0) cus = 256;
  int gc = 1;
  if (R <= 256) {
    if (H >= 3 && (long)n_rows * ((H + 3) / 4) >= 2L * cus)
      gc = 4;
    else if (H >= 2 && (long)n_rows * ((H + 1) / 2) >= 2L * cus)
      gc = 2;
  }
  dim3 grid(n_rows, (H + gc - 1) / gc);
  const size_t smem = (size_t)(gc * Dk + LA_WAVES * gc * (2 + R)) * sizeof(float);
  if (smem > 64 * 1024) JLLM_FAIL("latent attention: %zu bytes of LDS", smem);
  const size_t esz = dtype == JLLM_F32 ? 4 : 2;
  const int wide = (Dk % 4) == 0 && ((uintptr_t)cache % (4 * esz)) == 0;
#define LA_LAUNCH(GC)                                                                                              \
  latent_attention_generic_kernel<T, GC><<<grid, 64 * LA_WAVES, smem, stream>>>(                                   \
      (const T*)qa, ldq, (T*)out, ldo, (const T*)cache, block_table, max_blocks, row_req, positions, H, R, Dk, page_size, \
      window, scale, sink, wide)
  JLLM_DISPATCH_1(dtype, T, {
    if (gc == 4)
      LA_LAUNCH(4);
    else if (gc == 2)
      LA_LAUNCH(2);
    else
      LA_LAUNCH(1);
  })
#undef LA_LAUNCH
  JLLM_CHECK_LAUNCH("latent_attention_generic");
  return 0;
}

// Causal attention over a paged cache whose keys and values have sizes of their own, with the options that several
// designs put around the softmax: several score maps per head over shared values, a cap on the scores, a norm over a
// whole projection or over every head, rotation of neighbouring pairs or of a head's halves, a query scale that follows
// the position, a sliding window that may keep the first keys, a sink in the denominator, a gate per channel or per head.
// fp32 or bf16 storage, all arithmetic in fp32, any sizes. Three kernels:
//
//   qkv_prepare      one workgroup per row of the stacked projection [q | k | v]: optional RMS norm with gains over the
//                    whole of q and the whole of k (or over every head alone, with gains shared by the heads); optional
//                    rotation of the pairs (2i, 2i + 1) (or (i, i + rot_dims / 2)) among the first rot_dims entries of
//                    every q and k head by the row's position; optional q *= 1 + coef * ln(floor((p + 1) / every) + 1);
//                    q back in place, k and v into the row's place in the cache
//   attention_dv     one workgroup of four waves per (row, query slot). A query slot is one score map of one head: with
//                    M maps per head and H heads over G key/value heads there are H * M query slots and G * M key slots;
//                    query slot s reads key slot (s / (M * H / G)) * M + s % M and value head s / (M * H / G). Scores
//                    (q . k) * scale, then cap * tanh(score / cap) with a cap. Keys are walked in blocks of 64 aligned
//                    to absolute positions, wave w takes the blocks with c % 4 == w, the four waves' results are merged
//                    in wave order: a row's result depends only on its own position and keys. With a window the query
//                    at p sees keys p + 1 - window .. p and, with keep_first, the keys before keep_first (the blocks
//                    between them are passed over: their pages may be gone). A sink per head adds exp(sink) to the
//                    denominator and nothing to the sum
//   heads_finish     per (row, head): with two maps o = a1 - lambda * a2; optionally o / sqrt(mean(o^2) + eps) * gain;
//                    optionally times sigmoid(gate) or silu(gate) (a gate per channel or one per head), times a
//                    constant; written as the output product's
//                    input (other mixers whose heads end this way use it too)
//
// Cache layout of one layer run: keys [page][key slot][page_size][dk], values [page][value head][page_size][dv];
// position j of request r lives in page block_table[r][j / page_size] at offset j % page_size.
#include <math.h>

#include "common.h"

#define ADV_WAVES 4
#define ADV_MAX_ACC 8  // dv <= 512
#define PREP_THREADS 256

template <typename T, typename TG>
__global__ __launch_bounds__(PREP_THREADS) void qkv_prepare_kernel(
    T* __restrict__ qkv, int ld, const int* __restrict__ positions, const int* __restrict__ slots, int q_slots, int k_slots,
    int v_heads, int dk, int dv, const TG* __restrict__ gq, const TG* __restrict__ gk, float eps,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rot_dims, float temp_coef, int temp_every,
    T* __restrict__ kcache, T* __restrict__ vcache, int page_size, int norm_per_head, int pair_halves) {
  extern __shared__ float sm[];  // q and k of the row
  __shared__ float red[PREP_THREADS / 64];
  const int t = blockIdx.x;
  const int nq = q_slots * dk, nk = k_slots * dk, nv = v_heads * dv;
  T* row = qkv + (size_t)t * ld;
  const int pos = positions[t];
  for (int i = threadIdx.x; i < nq + nk; i += PREP_THREADS) sm[i] = ldf(row, i);
  __syncthreads();
  if (gq && norm_per_head) {  // every head alone, a wave per head; the gains [dk] are shared by the heads of q (of k)
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int head = wave; head < q_slots + k_slots; head += PREP_THREADS / 64) {
      float* p = sm + (size_t)head * dk;
      float ss = 0.f;
      for (int i = lane; i < dk; i += 64) ss = fmaf(p[i], p[i], ss);
      const float r = norm_scale(wave_sum(ss), dk, eps);
      const TG* g = head < q_slots ? gq : gk;
      for (int i = lane; i < dk; i += 64) p[i] = p[i] * r * ldf(g, i);
    }
    __syncthreads();
  } else if (gq) {  // the norm over a whole projection, before the heads are split
    float sq = 0.f, sk = 0.f;
    for (int i = threadIdx.x; i < nq; i += PREP_THREADS) sq = fmaf(sm[i], sm[i], sq);
    for (int i = threadIdx.x; i < nk; i += PREP_THREADS) sk = fmaf(sm[nq + i], sm[nq + i], sk);
    const float rq = norm_scale(block_sum<PREP_THREADS / 64>(sq, red), nq, eps);
    const float rk = norm_scale(block_sum<PREP_THREADS / 64>(sk, red), nk, eps);
    for (int i = threadIdx.x; i < nq; i += PREP_THREADS) sm[i] = sm[i] * rq * ldf(gq, i);
    for (int i = threadIdx.x; i < nk; i += PREP_THREADS) sm[nq + i] = sm[nq + i] * rk * ldf(gk, i);
    __syncthreads();
  }
  if (rot_dims > 0) {  // a thread owns a pair: nothing else reads or writes it
    const int half = rot_dims >> 1;
    const int pairs = (q_slots + k_slots) * half;
    for (int i = threadIdx.x; i < pairs; i += PREP_THREADS) {
      const int head = i / half, f = i % half;
      float* p = sm + (size_t)head * dk + (pair_halves ? f : 2 * f);
      const int other = pair_halves ? half : 1;  // the pair (f, f + half) or (2f, 2f + 1)
      const float c = cos_t[(size_t)pos * half + f], s = sin_t[(size_t)pos * half + f];
      const float u = p[0], v = p[other];
      p[0] = u * c - v * s;
      p[other] = v * c + u * s;
    }
    __syncthreads();
  }
  float temp = 1.0f;
  if (temp_every > 0) temp = 1.0f + temp_coef * logf((float)((pos + 1) / temp_every) + 1.0f);
  for (int i = threadIdx.x; i < nq; i += PREP_THREADS) stf(row, i, sm[i] * temp);
  const int slot = slots ? slots[t] : -1;
  if (slot < 0) return;  // a row that stores nothing (padding of a step of fixed size; a run that reads another's cache)
  const int page = slot / page_size, off = slot % page_size;
  for (int i = threadIdx.x; i < nk; i += PREP_THREADS) {
    const int h = i / dk, e = i % dk;
    stf(kcache, (((size_t)page * k_slots + h) * page_size + off) * dk + e, sm[nq + i]);
  }
  for (int i = threadIdx.x; i < nv; i += PREP_THREADS) {
    const int h = i / dv, e = i % dv;
    vcache[(((size_t)page * v_heads + h) * page_size + off) * dv + e] = row[nq + nk + i];
  }
}

extern "C" int jllm_qkv_prepare(void* qkv, int ld, int dtype, int n_tokens, const int* positions, const int* slots,
                                int q_slots, int k_slots, int v_heads, int dk, int dv, const void* gq, const void* gk,
                                int gain_dtype, float eps, const float* cos_t, const float* sin_t, int rot_dims,
                                float temp_coef, int temp_every, void* kcache, void* vcache, int page_size,
                                int norm_per_head, int pair_halves, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (q_slots <= 0 || k_slots <= 0 || v_heads <= 0 || dk <= 0 || dv <= 0) JLLM_FAIL("qkv_prepare: sizes %d %d %d %d %d", q_slots, k_slots, v_heads, dk, dv);
  if (ld < (q_slots + k_slots) * dk + v_heads * dv) JLLM_FAIL("qkv_prepare: rows of %d entries are shorter than q, k and v", ld);
  if ((gq == nullptr) != (gk == nullptr)) JLLM_FAIL("qkv_prepare: the norm takes gains for both q and k");
  if (rot_dims < 0 || rot_dims % 2 || rot_dims > dk || (rot_dims && (!cos_t || !sin_t))) JLLM_FAIL("qkv_prepare: a rotary width of %d for heads of %d", rot_dims, dk);
  if (page_size <= 0) JLLM_FAIL("qkv_prepare: page_size %d", page_size);
  const size_t smem = (size_t)(q_slots + k_slots) * dk * sizeof(float);
  if (smem > 64 * 1024) JLLM_FAIL("qkv_prepare: q and k of a row take %zu bytes of LDS (64 KB are taken)", smem);
  JLLM_DISPATCH_1(dtype, T, {
    JLLM_DISPATCH_1(gain_dtype, TG, {
      qkv_prepare_kernel<T, TG><<<n_tokens, PREP_THREADS, smem, stream>>>(
          (T*)qkv, ld, positions, slots, q_slots, k_slots, v_heads, dk, dv, (const TG*)gq, (const TG*)gk, eps, cos_t, sin_t,
          rot_dims, temp_coef, temp_every, (T*)kcache, (T*)vcache, page_size, norm_per_head, pair_halves);
    })
  })
  JLLM_CHECK_LAUNCH("qkv_prepare");
  return 0;
}

// ---------------------------------------------------------------------------------------------------------------------

template <typename T, typename TO>
__global__ __launch_bounds__(64 * ADV_WAVES) void attention_dv_generic_kernel(
    const T* __restrict__ q, int ldq, TO* __restrict__ out, int ldo, const T* __restrict__ kcache,
    const T* __restrict__ vcache, const int* __restrict__ block_table, int max_blocks, const int* __restrict__ row_req,
    const int* __restrict__ positions, int q_slots, int maps, int per_kv, int dk, int dv, int page_size, int window,
    float scale, float softcap, int keep_first, const float* __restrict__ sinks) {
  extern __shared__ float smem[];
  float* qs = smem;       // dk
  float* mg = smem + dk;  // ADV_WAVES x (2 + dv)
  const int t = blockIdx.x, s = blockIdx.y;
  const int vh = s / per_kv;              // per_kv = maps * heads / kv heads
  const int ks = vh * maps + s % maps;
  const int k_slots = (q_slots / per_kv) * maps, v_heads = q_slots / per_kv;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int pos = positions[t];
  const int* tbl = block_table + (size_t)row_req[t] * max_blocks;
  const int first = window > 0 ? max(0, pos + 1 - window) : 0;
  for (int i = threadIdx.x; i < dk; i += 64 * ADV_WAVES) qs[i] = ldf(q + (size_t)t * ldq + (size_t)s * dk, i);
  __syncthreads();
  const int nacc = (dv + 63) >> 6;
  float acc[ADV_MAX_ACC];
#pragma unroll
  for (int a = 0; a < ADV_MAX_ACC; ++a) acc[a] = 0.f;
  float m = -INFINITY, l = 0.f;
  // keys before `kept` stay visible whatever the window: then the walk starts at block 0 and passes over the blocks
  // between the kept keys and the window (block c still belongs to wave c % 4)
  const int kept = window > 0 ? min(keep_first, first) : 0;
  const int b_first = kept > 0 ? 0 : first >> 6;
  for (int blk = b_first + ((wave - b_first) & (ADV_WAVES - 1)); blk * 64 <= pos; blk += ADV_WAVES) {
    const int c0 = blk * 64;
    if (c0 + 63 < first && c0 >= kept) continue;
    const int kj = c0 + lane;
    const bool valid = (kj >= first || kj < kept) && kj <= pos;
    float sc = -INFINITY;
    int page = 0, off = 0;
    if (valid) {
      page = tbl[kj / page_size];
      off = kj % page_size;
      const T* kr = kcache + (((size_t)page * k_slots + ks) * page_size + off) * dk;
      float d = 0.f;
      for (int i = 0; i < dk; ++i) d = fmaf(qs[i], ldf(kr, i), d);
      sc = d * scale;
      if (softcap > 0.f) sc = softcap * tanhf(sc / softcap);
    }
    const float m_new = fmaxf(m, wave_max(sc));
    const float p = valid ? expf(sc - m_new) : 0.f;
    const float alpha = expf(m - m_new);
    l = l * alpha + wave_sum(p);
#pragma unroll
    for (int a = 0; a < ADV_MAX_ACC; ++a) acc[a] *= alpha;
    m = m_new;
    const int j0 = c0 < kept ? 0 : max(0, first - c0), j1 = min(63, pos - c0);
    for (int j = j0; j <= j1; ++j) {  // the block's values in ascending order of the keys
      if (c0 + j < first && c0 + j >= kept) continue;  // between the kept keys and the window: its page may be gone
      const float pj = __shfl(p, j, 64);
      const int pg = __shfl(page, j, 64), of = __shfl(off, j, 64);
      const T* vr = vcache + (((size_t)pg * v_heads + vh) * page_size + of) * dv;
#pragma unroll
      for (int a = 0; a < ADV_MAX_ACC; ++a) {
        const int d = lane + a * 64;
        if (a < nacc && d < dv) acc[a] = fmaf(pj, ldf(vr, d), acc[a]);
      }
    }
  }
  float* mine = mg + (size_t)wave * (2 + dv);
  if (lane == 0) {
    mine[0] = m;
    mine[1] = l;
  }
#pragma unroll
  for (int a = 0; a < ADV_MAX_ACC; ++a) {
    const int d = lane + a * 64;
    if (a < nacc && d < dv) mine[2 + d] = acc[a];
  }
  __syncthreads();
  if (wave != 0) return;
  for (int w = 1; w < ADV_WAVES; ++w) {  // merged in the order of the waves
    const float* theirs = mg + (size_t)w * (2 + dv);
    const float om = theirs[0], ol = theirs[1];
    if (ol == 0.f) continue;  // that wave had no key
    const float m_new = fmaxf(m, om);
    const float ca = expf(m - m_new), cb = expf(om - m_new);
    l = l * ca + ol * cb;
#pragma unroll
    for (int a = 0; a < ADV_MAX_ACC; ++a) {
      const int d = lane + a * 64;
      if (a < nacc && d < dv) acc[a] = acc[a] * ca + theirs[2 + d] * cb;
    }
    m = m_new;
  }
  if (sinks) l += expf(sinks[s / maps] - m);  // one more term of the denominator, with no value
  const float inv = 1.0f / l;
  TO* o = out + (size_t)t * ldo + (size_t)s * dv;
#pragma unroll
  for (int a = 0; a < ADV_MAX_ACC; ++a) {
    const int d = lane + a * 64;
    if (a < nacc && d < dv) stf(o, d, acc[a] * inv);
  }
}

// q [rows, ldq] holds q_slots x dk per row; out [rows, ldo] gets q_slots x dv per row
extern "C" int jllm_attention_dv_generic(const void* q, int ldq, int dtype, void* out, int ldo, int out_dtype,
                                         const void* kcache, const void* vcache, const int* block_table, int max_blocks,
                                         const int* row_req, const int* positions, int n_tokens, int heads, int kv_heads,
                                         int maps, int dk, int dv, int page_size, int window, float scale, float softcap,
                                         int keep_first, const float* sinks, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (heads <= 0 || kv_heads <= 0 || heads % kv_heads != 0 || maps <= 0) JLLM_FAIL("attention: %d query heads over %d kv heads with %d maps", heads, kv_heads, maps);
  if (dk <= 0 || dv <= 0 || dv > 64 * ADV_MAX_ACC || dk > 4096) JLLM_FAIL("attention: key size %d, value size %d (this kernel takes values up to %d)", dk, dv, 64 * ADV_MAX_ACC);
  const int q_slots = heads * maps;
  if (q_slots > 65535) JLLM_FAIL("attention: too many heads");
  if (page_size <= 0 || max_blocks <= 0 || window < 0 || keep_first < 0) JLLM_FAIL("attention: page_size %d max_blocks %d window %d, %d first keys kept", page_size, max_blocks, window, keep_first);
  if (ldq < q_slots * dk || ldo < q_slots * dv) JLLM_FAIL("attention: row strides %d/%d", ldq, ldo);
  dim3 grid(n_tokens, q_slots);
  const size_t smem = (size_t)(dk + ADV_WAVES * (2 + dv)) * sizeof(float);
  JLLM_DISPATCH_1(dtype, T, {
    JLLM_DISPATCH_1(out_dtype, TO, {
      attention_dv_generic_kernel<T, TO><<<grid, 64 * ADV_WAVES, smem, stream>>>(
          (const T*)q, ldq, (TO*)out, ldo, (const T*)kcache, (const T*)vcache, block_table, max_blocks, row_req, positions,
          q_slots, maps, maps * (heads / kv_heads), dk, dv, page_size, window, scale, softcap, keep_first, sinks);
    })
  })
  JLLM_CHECK_LAUNCH("attention_dv_generic");
  return 0;
}

// ---------------------------------------------------------------------------------------------------------------------

template <typename TA, typename TG, typename TW, typename TO>
__global__ __launch_bounds__(64) void heads_finish_kernel(const TA* __restrict__ att, int lda, int maps, int dv,
                                                          float lambda, int normed, float eps, float norm_mul,
                                                          const TW* __restrict__ gain, const TG* __restrict__ gate, int ldg,
                                                          int gate_fn, float out_mul, TO* __restrict__ out, int ldo,
                                                          int gate_per_head) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const TA* a = att + (size_t)t * lda + (size_t)h * maps * dv;
  float ss = 0.f;
  if (normed) {
    for (int j = lane; j < dv; j += 64) {
      float o = ldf(a, j);
      if (maps == 2) o = o - lambda * ldf(a, dv + j);
      ss = fmaf(o, o, ss);
    }
    ss = wave_sum(ss);
  }
  const float r = normed ? norm_scale(ss, dv, eps) * norm_mul : 1.0f;
  for (int j = lane; j < dv; j += 64) {
    float o = ldf(a, j);
    if (maps == 2) o = o - lambda * ldf(a, dv + j);
    o *= r;
    if (gain) o *= ldf(gain, j);
    if (gate) {
      const float z = ldf(gate + (size_t)t * ldg, gate_per_head ? (size_t)h : (size_t)h * dv + j);
      o *= (gate_fn == 1 ? z : 1.0f) / (1.0f + expf(-z));  // 0: sigmoid(z), 1: silu(z)
    }
    stf(out + (size_t)t * ldo, (size_t)h * dv + j, o * out_mul);
  }
}

// att [rows, lda]: heads x maps x dv per row; gate [rows, ldg]: heads x dv per row (`gate_per_head`: heads per row, one
// number for the whole head) or null; out [rows, ldo]
extern "C" int jllm_heads_finish(const void* att, int lda, int att_dtype, int n_tokens, int heads, int maps, int dv,
                                 float lambda, int normed, float eps, float norm_mul, const void* gain, int gain_dtype,
                                 const void* gate, int ldg, int gate_dtype, int gate_fn, float out_mul, void* out, int ldo, int out_dtype,
                                 int gate_per_head, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (heads <= 0 || heads > 65535 || dv <= 0 || (maps != 1 && maps != 2)) JLLM_FAIL("heads_finish: %d heads of %d with %d maps (one or two are taken)", heads, dv, maps);
  if (lda < heads * maps * dv || ldo < heads * dv || (gate && ldg < (gate_per_head ? heads : heads * dv))) JLLM_FAIL("heads_finish: short rows");
  if (gate_fn != 0 && gate_fn != 1) JLLM_FAIL("heads_finish: gate function %d (0 sigmoid and 1 silu are built)", gate_fn);
  dim3 grid(n_tokens, heads);
  JLLM_DISPATCH_1(att_dtype, TA, {
    JLLM_DISPATCH_1(gate_dtype, TG, {
      JLLM_DISPATCH_1(gain_dtype, TW, {
        JLLM_DISPATCH_1(out_dtype, TO, {
          heads_finish_kernel<TA, TG, TW, TO><<<grid, 64, 0, stream>>>((const TA*)att, lda, maps, dv, lambda, normed, eps, norm_mul,
                                                                      (const TW*)gain, (const TG*)gate, ldg, gate_fn, out_mul, (TO*)out, ldo,
                                                                      gate_per_head);
        })
      })
    })
  })
  JLLM_CHECK_LAUNCH("heads_finish");
  return 0;
}

// The same finish for heads whose attention was computed in key ranges that are not merged yet: `partial` [rows][heads x
// maps][splits][dv + 2] holds every range's unnormalised sums, its maximum (as an exponent of two) and its sum, as the
// matrix-core attention kernel leaves them (attention_dv_mfma.hip). Lane z holds range z's maximum and sum, so the
// ranges' weights are known after two wave reductions; merging here saves the launch of a merge kernel.
template <typename TG, typename TW, typename TO>
__global__ __launch_bounds__(64) void heads_finish_split_kernel(const float* __restrict__ partial, int splits, int maps,
                                                                int dv, float lambda, int normed, float eps, float norm_mul,
                                                                const TW* __restrict__ gain, const TG* __restrict__ gate,
                                                                int ldg, int gate_fn, float out_mul, TO* __restrict__ out,
                                                                int ldo, int gate_per_head, const float* __restrict__ sinks) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  float o[4] = {0.f, 0.f, 0.f, 0.f};  // dv <= 256
  for (int m = 0; m < maps; ++m) {
    const float* pr = partial + (((size_t)t * gridDim.y + h) * maps + m) * splits * (dv + 2);
    const float mz = lane < splits ? pr[(size_t)lane * (dv + 2) + dv] : -INFINITY;
    const float lz = lane < splits ? pr[(size_t)lane * (dv + 2) + dv + 1] : 0.f;
    const float mx = wave_max(mz);
    const float wz = mz == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mz - mx);
    // a sink is one more term of the denominator: exp(sink) on the scale of the ranges' common maximum
    const float sink_term = sinks ? __builtin_amdgcn_exp2f(sinks[h] * 1.4426950408889634f - mx) : 0.f;
    const float inv = 1.0f / (wave_sum(lz * wz) + sink_term);
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      const int j = lane + 64 * jj;
      if (j >= dv) continue;
      float acc = 0.f;
#pragma unroll 4
      for (int z = 0; z < splits; ++z) {
        const float w = __shfl(wz, z, 64);
        const float v = pr[(size_t)z * (dv + 2) + j];
        acc = w != 0.f ? fmaf(v, w, acc) : acc;  // a range without keys left its sums unwritten
      }
      o[jj] = m == 0 ? acc * inv : o[jj] - lambda * (acc * inv);
    }
  }
  float ss = 0.f;
  if (normed) {
#pragma unroll
    for (int jj = 0; jj < 4; ++jj)
      if (lane + 64 * jj < dv) ss = fmaf(o[jj], o[jj], ss);
    ss = wave_sum(ss);
  }
  const float r = normed ? norm_scale(ss, dv, eps) * norm_mul : 1.0f;
#pragma unroll
  for (int jj = 0; jj < 4; ++jj) {
    const int j = lane + 64 * jj;
    if (j >= dv) continue;
    float v = o[jj] * r;
    if (gain) v *= ldf(gain, j);
    if (gate) {
      const float z = ldf(gate + (size_t)t * ldg, gate_per_head ? (size_t)h : (size_t)h * dv + j);
      v *= (gate_fn == 1 ? z : 1.0f) / (1.0f + expf(-z));
    }
    stf(out + (size_t)t * ldo, (size_t)h * dv + j, v * out_mul);
  }
}

extern "C" int jllm_heads_finish_split(const float* partial, int splits, int n_tokens, int heads, int maps, int dv, float lambda,
                                       int normed, float eps, float norm_mul, const void* gain, int gain_dtype, const void* gate,
                                       int ldg, int gate_dtype, int gate_fn, float out_mul, void* out, int ldo, int out_dtype,
                                       int gate_per_head, const float* sinks, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (heads <= 0 || heads > 65535 || dv <= 0 || dv > 256 || (maps != 1 && maps != 2) || splits < 1 || splits > 64)
    JLLM_FAIL("heads_finish: %d heads of %d with %d maps in %d key ranges", heads, dv, maps, splits);
  if (ldo < heads * dv || (gate && ldg < (gate_per_head ? heads : heads * dv))) JLLM_FAIL("heads_finish: short rows");
  if (gate_fn != 0 && gate_fn != 1) JLLM_FAIL("heads_finish: gate function %d (0 sigmoid and 1 silu are built)", gate_fn);
  if (sinks && maps != 1) JLLM_FAIL("heads_finish: a sink with %d maps per head", maps);
  dim3 grid(n_tokens, heads);
  JLLM_DISPATCH_1(gate_dtype, TG, {
    JLLM_DISPATCH_1(gain_dtype, TW, {
      JLLM_DISPATCH_1(out_dtype, TO, {
        heads_finish_split_kernel<TG, TW, TO><<<grid, 64, 0, stream>>>(partial, splits, maps, dv, lambda, normed, eps, norm_mul,
                                                                      (const TW*)gain, (const TG*)gate, ldg, gate_fn, out_mul,
                                                                      (TO*)out, ldo, gate_per_head, sinks);
      })
    })
  })
  JLLM_CHECK_LAUNCH("heads_finish_split");
  return 0;
}

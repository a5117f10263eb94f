// A gated delta rule with short causal convolutions in front: a recurrent mixer whose per-request state is one matrix
// per head (fp32) and the last taps - 1 inputs of every convolved channel. fp32 or bf16 activations, all arithmetic in
// fp32. A request's rows of a step are consecutive and in order (row_req ascends), so every kernel finds a request's
// rows in the step by itself and the same launches serve portions of prompts, single rows and steps of fixed size.
//
//   short_conv_silu      y[t, c] = silu(sum_j taps[c, K - 1 - j] x[t - j, c] (+ bias[c])); inputs before the step's first row of a
//                        request come from that request's state, inputs before position 0 are the state's zeros
//   short_conv_advance   the state's K - 1 inputs per channel move on by the request's rows of this step
//   delta_prepare        per (row, key head), what the recurrence would otherwise compute in every lane of every wave:
//                          q <- q / sqrt(sum q^2 + 1e-6) / sqrt(dk), k <- k / sqrt(sum k^2 + 1e-6), q . k, and per head
//                          beta = sigmoid(b), g = exp(-exp(A_log) * softplus(a + dt_bias)); all in fp32
//   gated_delta          token by token, with S [dk, dv] in registers:
//                          S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
//                        computed as  S^T k and S^T q of the old S in one pass, o = g S^T q + (k . q) u.
//                        The columns of S never meet: column j only needs v[j]. A workgroup of four waves owns 16 value
//                        columns of one head of one request: a wave 4 of them, 16 lanes per column with a sixteenth of
//                        the key rows each (sums over a column's lanes are moves inside a row of 16 lanes). It walks
//                        the request's rows in chunks of 16 that are requested a chunk ahead and shared through LDS.
//                        One request and 16 heads of 128 x 128 are 512 waves. The read-out o goes out raw in fp32; the
//                        heads' norm, gain and gate need all columns of a head and are the finishing kernel's
//                        (attention_dv.hip).
#include <math.h>

#include "common.h"

#define CONV_MAX_TAPS 16
#define GDR_COLS 16    // value columns of a workgroup (4 per wave)
#define GDR_PARTS 16   // lanes per column: each owns a sixteenth of the key rows
#define GDR_CHUNK 16   // rows staged at a time

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }

template <typename T, typename TW>
__global__ __launch_bounds__(256) void short_conv_silu_kernel(const T* __restrict__ x, int ldx, T* __restrict__ y, int ldy,
                                                              int channels, int taps, const TW* __restrict__ w,
                                                              const TW* __restrict__ bias, const float* __restrict__ state,
                                                              const int* __restrict__ row_req,
                                                              const int* __restrict__ state_slots) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= channels) return;
  const int req = row_req[t];
  int m = 0;  // rows of the same request in front of this one, as far as the taps reach
  while (m < taps - 1 && t - m - 1 >= 0 && row_req[t - m - 1] == req) ++m;
  const float* st = state + (size_t)state_slots[req] * (taps - 1) * channels;
  float acc = 0.f;
  const float shift = bias ? ldf(bias, c) : 0.f;
  for (int j = taps - 1; j >= 0; --j) {  // oldest input first
    float v;
    if (j <= m)
      v = ldf(x + (size_t)(t - j) * ldx, c);
    else
      v = st[(size_t)(taps - 1 - (j - m)) * channels + c];
    acc = fmaf(ldf(w, (size_t)c * taps + (taps - 1 - j)), v, acc);
  }
  stf(y + (size_t)t * ldy, c, silu_f(acc + shift));
}

// first row and number of rows of request `req` in the ascending list row_req[0 .. n)
__device__ __forceinline__ void rows_of_request(const int* __restrict__ row_req, int n, int req, int& lo, int& cnt) {
  if (req < n) {
    // a step of single rows has request r's one row at place r: three loads side by side in place of two searches.
    // In an ascending list, a place that holds r between two neighbours that do not is all of r's rows.
    const int here = row_req[req];
    const int before = req > 0 ? row_req[req - 1] : -1;
    const int after = req + 1 < n ? row_req[req + 1] : 0x7fffffff;
    if (here == req && before != req && after != req) {
      lo = req;
      cnt = 1;
      return;
    }
  }
  int a = 0, b = n;
  while (a < b) {
    const int mid = (a + b) >> 1;
    if (row_req[mid] < req) a = mid + 1; else b = mid;
  }
  lo = a;
  b = n;
  while (a < b) {
    const int mid = (a + b) >> 1;
    if (row_req[mid] <= req) a = mid + 1; else b = mid;
  }
  cnt = a - lo;
}

template <typename T>
__global__ __launch_bounds__(256) void short_conv_advance_kernel(const T* __restrict__ x, int ldx, int channels, int taps,
                                                                 float* __restrict__ state, const int* __restrict__ row_req,
                                                                 int n_rows, const int* __restrict__ state_slots) {
  const int req = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= channels) return;
  int lo, n;
  rows_of_request(row_req, n_rows, req, lo, n);
  if (n == 0) return;
  float* st = state + (size_t)state_slots[req] * (taps - 1) * channels;
  float keep[CONV_MAX_TAPS];
#pragma unroll
  for (int i = 0; i < CONV_MAX_TAPS; ++i) {
    if (i >= taps - 1) break;
    const int at = n - (taps - 1) + i;  // which input of this step, counted from the request's first row
    keep[i] = at >= 0 ? ldf(x + (size_t)(lo + at) * ldx, c) : st[(size_t)(taps - 1 + at) * channels + c];
  }
#pragma unroll
  for (int i = 0; i < CONV_MAX_TAPS; ++i) {
    if (i >= taps - 1) break;
    st[(size_t)i * channels + c] = keep[i];
  }
}

extern "C" int jllm_short_conv(const void* x, int ldx, void* y, int ldy, int dtype, int n_rows, int n_requests, int channels,
                               int taps, const void* w, const void* bias, int w_dtype, float* state, const int* row_req,
                               const int* state_slots, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (channels <= 0 || taps < 1 || taps > CONV_MAX_TAPS) JLLM_FAIL("short_conv: %d channels, %d taps (1..%d taps are taken)", channels, taps, CONV_MAX_TAPS);
  if (ldx < channels || ldy < channels || n_requests <= 0 || n_requests > n_rows) JLLM_FAIL("short_conv: rows %d/%d of %d channels, %d requests in %d rows", ldx, ldy, channels, n_requests, n_rows);
  const int cb = (channels + 255) / 256;
  JLLM_DISPATCH_1(dtype, T, {
    JLLM_DISPATCH_1(w_dtype, TW, {
      short_conv_silu_kernel<T, TW><<<dim3(n_rows, cb), 256, 0, stream>>>((const T*)x, ldx, (T*)y, ldy, channels, taps, (const TW*)w,
                                                                          (const TW*)bias, state, row_req, state_slots);
    })
    if (taps > 1)
      short_conv_advance_kernel<T><<<dim3(n_requests, cb), 256, 0, stream>>>((const T*)x, ldx, channels, taps, state, row_req,
                                                                             n_rows, state_slots);
  })
  JLLM_CHECK_LAUNCH("short_conv");
  return 0;
}

// ---------------------------------------------------------------------------------------------------------------------

// prep row: qn (kv_heads x dk) | kn (kv_heads x dk) | g (heads) | beta (heads) | q . k (kv_heads) | g per key channel
// (heads x dk, only with `decay_rows`: the decay's input per head and key channel, fp32 [rows, ldd], with dt_bias of
// heads x dk entries; the one number per head is then not written)
template <typename T, typename TW>
__global__ __launch_bounds__(64) void delta_prepare_kernel(const T* __restrict__ conv, int ldc, const T* __restrict__ proj,
                                                           int ldp, int a_off, int b_off, const TW* __restrict__ a_log,
                                                           const TW* __restrict__ dt_bias, float* __restrict__ prep, int ldq,
                                                           int heads, int kv_heads, int dk,
                                                           const float* __restrict__ decay_rows, int ldd) {
  const int row = blockIdx.x, g = blockIdx.y, lane = threadIdx.x;
  const T* q = conv + (size_t)row * ldc + (size_t)g * dk;
  const T* k = conv + (size_t)row * ldc + (size_t)(kv_heads + g) * dk;
  float sq = 0.f, sk = 0.f, qk = 0.f;
  for (int i = lane; i < dk; i += 64) {
    const float a = ldf(q, i), b = ldf(k, i);
    sq = fmaf(a, a, sq);
    sk = fmaf(b, b, sk);
    qk = fmaf(a, b, qk);
  }
  sq = wave_sum(sq), sk = wave_sum(sk), qk = wave_sum(qk);
  const float rq = (1.0f / sqrtf((float)dk)) / sqrtf(sq + 1e-6f), rk = 1.0f / sqrtf(sk + 1e-6f);
  float* out = prep + (size_t)row * ldq;
  for (int i = lane; i < dk; i += 64) {
    out[(size_t)g * dk + i] = ldf(q, i) * rq;
    out[(size_t)(kv_heads + g) * dk + i] = ldf(k, i) * rk;
  }
  const int per = heads / kv_heads;
  float* tail = out + (size_t)2 * kv_heads * dk;
  for (int j = lane; j < per; j += 64) {
    const int h = g * per + j;
    if (!decay_rows) {
      const float z = ldf(proj + (size_t)row * ldp, a_off + h) + ldf(dt_bias, h);
      const float sp = z > 20.f ? z : log1pf(expf(z));
      tail[h] = expf(-expf(ldf(a_log, h)) * sp);
    }
    tail[heads + h] = 1.0f / (1.0f + expf(-ldf(proj + (size_t)row * ldp, b_off + h)));
  }
  if (lane == 0) tail[2 * heads + g] = qk * rq * rk;
  if (decay_rows) {
    float* gv = tail + 2 * heads + kv_heads;
    for (int j = 0; j < per; ++j) {
      const int h = g * per + j;
      const float rate = expf(ldf(a_log, h));
      for (int i = lane; i < dk; i += 64) {
        const float z = decay_rows[(size_t)row * ldd + (size_t)h * dk + i] + ldf(dt_bias, (size_t)h * dk + i);
        const float sp = z > 20.f ? z : log1pf(expf(z));
        gv[(size_t)h * dk + i] = expf(-rate * sp);
      }
    }
  }
}

struct GdrArgs {
  const void* conv;   // [rows, ldc]: q | k | v (heads x dv) convolved; only v is read here
  int ldc;
  const float* prep;  // [rows, ldq]: what delta_prepare left
  int ldq;
  float* state;       // [slots, heads, dv, dk]: a head's matrix column by column
  float* out;         // [rows, ldo]: heads x dv, the raw read-out
  int ldo;
  const int* row_req;
  const int* state_slots;
  int n_rows, heads, kv_heads, dk, dv;
};

__device__ __forceinline__ float row16_sum(float d) {  // over a row of 16 lanes, left in all of them
  d += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, d), 0xB1, 0xF, 0xF, true));
  d += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, d), 0x4E, 0xF, 0xF, true));
  d += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, d), 0x141, 0xF, 0xF, true));
  d += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, d), 0x140, 0xF, 0xF, true));
  return d;
}

// thread = wave * 64 + c * 16 + part: column blockIdx.z * 16 + wave * 4 + c, key rows part * E .. + E
// CHANNEL: the decay is a vector over the key channels (S's rows) instead of one number per head:
//   S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q = (diag(g) S_old)^T q + (k . q) u
// FEW: the form for steps of few rows per request (decoding). It leaves out the interleaved walk over a full chunk, whose
// registers would halve the workgroups that a compute unit holds: such a step is a wait for each request's state, and
// the more workgroups wait at once, the more of it is in flight. A token's arithmetic is the same in both forms.
template <typename T, int E, bool CHANNEL, bool FEW>
__global__ __launch_bounds__(256) void gated_delta_kernel(GdrArgs A) {
  constexpr int C = GDR_CHUNK;
  constexpr int DKP = GDR_PARTS * E;              // the key size, padded with zeros
  constexpr int NV = CHANNEL ? 3 : 2;             // vectors over the key size per row: q | k (| g)
  constexpr int ROWF = NV * DKP + GDR_COLS + 4;   // q | k (| g) | v of the workgroup's columns | g | beta | q . k | -
  constexpr int NJ = C * DKP / 256;               // entries of one vector of a chunk per thread
  constexpr int NQK = NV * NJ;
  __shared__ __align__(16) float sm[C * ROWF];
  const int tid = threadIdx.x;
  const int part = tid & 15, cw = tid >> 4;  // cw: the column within the workgroup
  const int req = blockIdx.x, h = blockIdx.y;
  const int col0 = blockIdx.z * GDR_COLS;
  const int col = col0 + cw;
  const bool col_on = col < A.dv;
  int lo, n;
  rows_of_request(A.row_req, A.n_rows, req, lo, n);
  if (n == 0) return;
  const int dk = A.dk;
  const int kvh = h / (A.heads / A.kv_heads);
  const int i0 = part * E;
  float* S_at = A.state + ((size_t)A.state_slots[req] * A.heads + h) * dk * A.dv;
  float S[E];
  // A head's state lies column by column ([dv][dk]), so a lane's entries are side by side and a workgroup's 16 columns one
  // run of memory. Every lane loads from a place that exists and drops what it does not own: a load inside a condition
  // waits for the loads before it (its register is also written on the other path), and these would come one by one.
  const bool wide = E >= 4 && (dk & 3) == 0;  // then a lane's entries start on 16 bytes and end with the column
  if (wide) {
#pragma unroll
    for (int e = 0; e < E; e += 4) {
      const bool own = col_on && i0 + e < dk;
      const float4 s = *reinterpret_cast<const float4*>(S_at + (own ? (size_t)col * dk + i0 + e : 0));
      S[e] = own ? s.x : 0.f;
      S[(e + 1) % E] = own ? s.y : 0.f;
      S[(e + 2) % E] = own ? s.z : 0.f;
      S[(e + 3) % E] = own ? s.w : 0.f;
    }
  } else {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const bool own = col_on && i0 + e < dk;
      const float s = S_at[own ? (size_t)col * dk + i0 + e : 0];
      S[e] = own ? s : 0.f;
    }
  }
  const T* conv = (const T*)A.conv;
  const size_t q_at = (size_t)kvh * dk, k_at = (size_t)(A.kv_heads + kvh) * dk;
  const size_t tail_at = (size_t)2 * A.kv_heads * dk;
  const size_t g_at = tail_at + 2 * A.heads + A.kv_heads + (size_t)h * dk;
  const size_t v_at = (size_t)2 * A.kv_heads * dk + (size_t)h * A.dv + col0;
  float rqk[NQK], rv, rs;
  auto request = [&](int r0) {  // rows r0 .. r0 + C of the request, as far as it has them
    const int have = min(C, n - r0);
#pragma unroll
    for (int v = 0; v < NV; ++v) {  // vector by vector, so that every index below is a shift and a mask
      const size_t at = v == 0 ? q_at : v == 1 ? k_at : g_at;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int idx = tid + 256 * j;
        const int t = idx / DKP, i = idx % DKP;
        const bool own = t < have && i < dk;
        const float p = A.prep[(size_t)(lo + r0 + (own ? t : 0)) * A.ldq + at + (own ? i : 0)];
        rqk[v * NJ + j] = own ? p : 0.f;
      }
    }
    {
      const int t = tid / GDR_COLS, cc = tid % GDR_COLS;
      const bool own = t < have && col0 + cc < A.dv;
      const float p = ldf(conv + (size_t)(lo + r0 + (own ? t : 0)) * A.ldc + v_at, own ? cc : 0);
      rv = own ? p : 0.f;
    }
    {
      const int which = tid % 3;  // g, beta, q . k
      const bool own = tid < 3 * C && tid / 3 < have;
      const float p = A.prep[(size_t)(lo + r0 + (own ? tid / 3 : 0)) * A.ldq + tail_at + (which == 0 ? h : which == 1 ? A.heads + h : 2 * A.heads + kvh)];
      rs = own ? p : 0.f;
    }
  };
  auto stage = [&]() {
#pragma unroll
    for (int v = 0; v < NV; ++v) {
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int idx = tid + 256 * j;
        sm[(idx / DKP) * ROWF + v * DKP + idx % DKP] = rqk[v * NJ + j];
      }
    }
    sm[(tid / GDR_COLS) * ROWF + NV * DKP + tid % GDR_COLS] = rv;
    if (tid < 3 * C) sm[(tid / 3) * ROWF + NV * DKP + GDR_COLS + tid % 3] = rs;
  };
  request(0);
  for (int r0 = 0; r0 < n; r0 += C) {
    __syncthreads();  // the chunk before has been read
    stage();
    __syncthreads();
    if (r0 + C < n) request(r0 + C);  // in flight while this chunk is worked through
    const int have = min(C, n - r0);
    // One token: the lane's rows of S move on; what it leaves are the lane's part of S^T q and (q . k) u. Only the sum
    // behind u (S^T k over the lanes) stands between one token and the next, in two chains of multiply-adds; the
    // read-out's sum over the lanes is taken afterwards, for a full chunk for all its tokens together. A token's
    // arithmetic is the same sequence in a full chunk and in a short one.
    auto token = [&](int t, float& sq_part, float& qu) {
      const float* row = sm + t * ROWF;
      float q[E], k[E];
#pragma unroll
      for (int e = 0; e < E; ++e) {
        q[e] = row[i0 + e];
        k[e] = row[DKP + i0 + e];
      }
      const float v = row[NV * DKP + cw], g = row[NV * DKP + GDR_COLS], beta = row[NV * DKP + GDR_COLS + 1];
      const float qk = row[NV * DKP + GDR_COLS + 2];
      float sk0 = 0.f, sk1 = 0.f, sq_ = 0.f;
      if constexpr (CHANNEL) {
#pragma unroll
        for (int e = 0; e < E; ++e) S[e] *= row[2 * DKP + i0 + e];
      }
#pragma unroll
      for (int e = 0; e < E; e += 2) {
        sk0 = fmaf(S[e], k[e], sk0);
        sk1 = fmaf(S[e + 1], k[e + 1], sk1);
      }
#pragma unroll
      for (int e = 0; e < E; ++e) sq_ = fmaf(S[e], q[e], sq_);
      const float sk_ = row16_sum(sk0 + sk1);
      if constexpr (CHANNEL) {
        const float u = beta * (v - sk_);
#pragma unroll
        for (int e = 0; e < E; ++e) S[e] = fmaf(k[e], u, S[e]);
        qu = u;
      } else {
        const float u = beta * (v - g * sk_);
#pragma unroll
        for (int e = 0; e < E; ++e) S[e] = fmaf(k[e], u, g * S[e]);
        qu = qk * u;
      }
      sq_part = sq_;
    };
    auto read_out = [&](int t, float sq_sum, float qu) {  // o = S^T q after the token's write
      if constexpr (CHANNEL) return fmaf(sm[t * ROWF + NV * DKP + GDR_COLS + 2], qu, sq_sum);  // (q . k) u + S^T q
      return fmaf(sm[t * ROWF + NV * DKP + GDR_COLS], sq_sum, qu);
    };
    if (!FEW && have == C) {
      float sq[C], qu[C];
#pragma unroll
      for (int t = 0; t < C; ++t) token(t, sq[t], qu[t]);
#pragma unroll
      for (int t = 0; t < C; ++t) sq[t] = read_out(t, row16_sum(sq[t]), qu[t]);
      float mine = sq[0];  // lane `part` of a column writes token `part`
#pragma unroll
      for (int t = 1; t < C; ++t) mine = part == t ? sq[t] : mine;
      if (col_on) A.out[(size_t)(lo + r0 + part) * A.ldo + (size_t)h * A.dv + col] = mine;
    } else {
      for (int t = 0; t < have; ++t) {
        float sq_part, qu;
        token(t, sq_part, qu);
        const float o = read_out(t, row16_sum(sq_part), qu);
        if (part == 0 && col_on) A.out[(size_t)(lo + r0 + t) * A.ldo + (size_t)h * A.dv + col] = o;
      }
    }
  }
  if (wide) {
#pragma unroll
    for (int e = 0; e < E; e += 4)
      if (col_on && i0 + e < dk)
        *reinterpret_cast<float4*>(S_at + (size_t)col * dk + i0 + e) = make_float4(S[e], S[(e + 1) % E], S[(e + 2) % E], S[(e + 3) % E]);
  } else {
#pragma unroll
    for (int e = 0; e < E; ++e)
      if (col_on && i0 + e < dk) S_at[(size_t)col * dk + i0 + e] = S[e];
  }
}

// prep: fp32 scratch [rows, >= 2 kv_heads dk + 2 heads + kv_heads (+ heads dk with decay_rows)]. decay_rows: null (one
// decay per head, from proj at a_off, dt_bias of heads entries) or fp32 [rows, ldd] with the decay's input per head and
// key channel (dt_bias of heads x dk entries)
extern "C" int jllm_gated_delta(const void* qkv, int ldc, const void* proj, int ldp, int a_off, int b_off, int dtype,
                                const void* a_log, const void* dt_bias, int w_dtype, float* prep, int ldq, float* state,
                                float* out, int ldo, const int* row_req, const int* state_slots, int n_rows, int n_requests,
                                int heads, int kv_heads, int dk, int dv, const float* decay_rows, int ldd,
                                hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (heads <= 0 || kv_heads <= 0 || heads % kv_heads || heads > 65535) JLLM_FAIL("gated_delta: %d heads over %d key heads", heads, kv_heads);
  if (dk <= 0 || dk > GDR_PARTS * 16 || dv <= 0 || dv > GDR_COLS * 65535) JLLM_FAIL("gated_delta: key size %d (1..%d are taken), value size %d", dk, GDR_PARTS * 16, dv);
  if (n_requests <= 0 || n_requests > n_rows) JLLM_FAIL("gated_delta: %d requests in %d rows", n_requests, n_rows);
  const bool channel = decay_rows != nullptr;
  if (ldc < 2 * kv_heads * dk + heads * dv || ldo < heads * dv || (!channel && (ldp < a_off + heads || a_off < 0)) ||
      ldp < b_off + heads || b_off < 0 || ldq < 2 * kv_heads * dk + 2 * heads + kv_heads + (channel ? heads * dk : 0) ||
      (channel && ldd < heads * dk))
    JLLM_FAIL("gated_delta: short rows");
  JLLM_DISPATCH_1(dtype, T, {
    JLLM_DISPATCH_1(w_dtype, TW, {
      delta_prepare_kernel<T, TW><<<dim3(n_rows, kv_heads), 64, 0, stream>>>((const T*)qkv, ldc, (const T*)proj, ldp, a_off, b_off,
                                                                            (const TW*)a_log, (const TW*)dt_bias, prep, ldq, heads,
                                                                            kv_heads, dk, decay_rows, ldd);
    })
  })
  GdrArgs A{qkv, ldc, prep, ldq, state, out, ldo, row_req, state_slots, n_rows, heads, kv_heads, dk, dv};
  dim3 grid(n_requests, heads, (dv + GDR_COLS - 1) / GDR_COLS);
  const int per_lane = (dk + GDR_PARTS - 1) / GDR_PARTS;
  const bool few = n_rows <= 2 * n_requests;
#define GDR_LAUNCH(E)                                                           \
  do {                                                                          \
    if (channel && few)                                                         \
      gated_delta_kernel<T, E, true, true><<<grid, 256, 0, stream>>>(A);        \
    else if (channel)                                                           \
      gated_delta_kernel<T, E, true, false><<<grid, 256, 0, stream>>>(A);       \
    else if (few)                                                               \
      gated_delta_kernel<T, E, false, true><<<grid, 256, 0, stream>>>(A);       \
    else                                                                        \
      gated_delta_kernel<T, E, false, false><<<grid, 256, 0, stream>>>(A);      \
  } while (0)
  JLLM_DISPATCH_1(dtype, T, {
    if (per_lane <= 2)
      GDR_LAUNCH(2);
    else if (per_lane <= 4)
      GDR_LAUNCH(4);
    else if (per_lane <= 8)
      GDR_LAUNCH(8);
    else
      GDR_LAUNCH(16);
  })
#undef GDR_LAUNCH
  JLLM_CHECK_LAUNCH("gated_delta");
  return 0;
}

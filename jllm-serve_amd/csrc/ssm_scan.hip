// A selective state-space recurrence (the Mamba-2 form: one decay per head and token) and the gated norm behind it.
// fp32 or bf16 activations, all arithmetic and the state in fp32. A request's rows of a step are consecutive and in
// order (row_req ascends), so the kernel finds a request's rows by itself and the same launch serves portions of
// prompts, single rows and steps of fixed size.
//
//   ssm_scan          per head, token by token, with S [n, dv] (n: state size) in registers:
//                       dt = softplus(dt_in + dt_bias);  S <- exp(-exp(A_log) dt) S + dt B x^T;  y = S^T C + D x
//                     B and C [groups x n] are shared by the heads of a group. The columns of S never meet (column j
//                     only needs x[j]), so a workgroup of four waves owns 16 value columns of one head of one request:
//                     16 lanes per column with a sixteenth of the state rows each; sums over a column's lanes are moves
//                     inside a row of 16 lanes. Rows are requested in chunks of 16 a chunk ahead and shared through
//                     LDS; dt and the decay of a chunk's rows are computed once per chunk by 16 lanes. A token's
//                     arithmetic is one sequence of operations whatever the cut of the prompt (the tokens of a full
//                     chunk are only interleaved, their sums over the lanes taken together), so fp32 results do not
//                     depend on it.
//   gated_group_norm  out = rmsnorm_g(y * silu(z)) * w: the gate comes first, then every one of `groups` equal parts
//                     of a row is divided by its own root mean square
#include <math.h>

#include "common.h"

#define SSM_COLS 16
#define SSM_PARTS 16
#define SSM_CHUNK 16

struct SsmArgs {
  const void* xbc;    // [rows, ld]: x (heads x dv) | B (groups x n) | C (groups x n), convolved
  int ld;
  const void* dt;     // [rows, ldt], heads entries from dt_off on
  int ldt, dt_off;
  const void* a_log;  // [heads]
  const void* dt_bias;
  const void* skip;   // D [heads]
  float* state;       // [slots, heads, dv, n]: a head's matrix column by column
  float* out;         // [rows, ldo]: heads x dv
  int ldo;
  const int* row_req;
  const int* state_slots;
  int n_rows, heads, groups, n, dv;
};

__device__ __forceinline__ void ssm_rows_of_request(const int* __restrict__ row_req, int n, int req, int& lo, int& cnt) {
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

__device__ __forceinline__ float ssm_row16_sum(float d) {  // over a row of 16 lanes, left in all of them
  d += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, d), 0xB1, 0xF, 0xF, true));
  d += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, d), 0x4E, 0xF, 0xF, true));
  d += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, d), 0x141, 0xF, 0xF, true));
  d += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, d), 0x140, 0xF, 0xF, true));
  return d;
}

// thread = cw * 16 + part: column blockIdx.z * 16 + cw, state rows part * E .. + E
// FEW: the form for steps of few rows per request (decoding). It leaves out the interleaved walk over a full chunk, whose
// registers would halve the workgroups that a compute unit holds: such a step is a wait for each request's state, and
// the more workgroups wait at once, the more of it is in flight. A token's arithmetic is the same in both forms.
template <typename T, typename TW, int E, bool FEW>
__global__ __launch_bounds__(256) void ssm_scan_kernel(SsmArgs A) {
  constexpr int C = SSM_CHUNK;
  constexpr int NP = SSM_PARTS * E;            // the state size, padded with zeros
  constexpr int ROWF = 2 * NP + SSM_COLS + 4;  // B | C | x of the workgroup's columns | dt | decay | - | -
  constexpr int NBC = C * 2 * NP / 256;
  __shared__ __align__(16) float sm[C * ROWF];
  const int tid = threadIdx.x;
  const int part = tid & 15, cw = tid >> 4;
  const int req = blockIdx.x, h = blockIdx.y;
  const int col0 = blockIdx.z * SSM_COLS;
  const int col = col0 + cw;
  const bool col_on = col < A.dv;
  int lo, n;
  ssm_rows_of_request(A.row_req, A.n_rows, req, lo, n);
  if (n == 0) return;
  const int ns = A.n;
  const int grp = h / (A.heads / A.groups);
  const int i0 = part * E;
  float* S_at = A.state + ((size_t)A.state_slots[req] * A.heads + h) * ns * A.dv;
  float S[E];
  // A head's state lies column by column ([dv][ns]), so a lane's entries are side by side and a workgroup's 16 columns one
  // run of memory. Every lane loads from a place that exists and drops what it does not own: a load inside a condition
  // waits for the loads before it (its register is also written on the other path), and these would come one by one.
  const bool wide = E >= 4 && (ns & 3) == 0;  // then a lane's entries start on 16 bytes and end with the column
  if (wide) {
#pragma unroll
    for (int e = 0; e < E; e += 4) {
      const bool own = col_on && i0 + e < ns;
      const float4 s = *reinterpret_cast<const float4*>(S_at + (own ? (size_t)col * ns + i0 + e : 0));
      S[e] = own ? s.x : 0.f;
      S[(e + 1) % E] = own ? s.y : 0.f;
      S[(e + 2) % E] = own ? s.z : 0.f;
      S[(e + 3) % E] = own ? s.w : 0.f;
    }
  } else {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const bool own = col_on && i0 + e < ns;
      const float s = S_at[own ? (size_t)col * ns + i0 + e : 0];
      S[e] = own ? s : 0.f;
    }
  }
  const T* xbc = (const T*)A.xbc;
  const T* dtp = (const T*)A.dt;
  const size_t inner = (size_t)A.heads * A.dv;
  const size_t b_at = inner + (size_t)grp * ns, c_at = inner + (size_t)(A.groups + grp) * ns;
  const size_t x_at = (size_t)h * A.dv + col0;
  const float rate = expf(ldf((const TW*)A.a_log, h)), shift = ldf((const TW*)A.dt_bias, h), skip = ldf((const TW*)A.skip, h);
  float rbc[NBC], rx, rdt;
  auto request = [&](int r0) {
    const int have = min(C, n - r0);
#pragma unroll
    for (int j = 0; j < NBC; ++j) {
      const int idx = tid + 256 * j;
      const int t = idx / (2 * NP), w = idx % (2 * NP);
      const int i = w % NP;
      const bool own = t < have && i < ns;
      const float p = ldf(xbc + (size_t)(lo + r0 + (own ? t : 0)) * A.ld + (w < NP ? b_at : c_at), own ? i : 0);
      rbc[j] = own ? p : 0.f;
    }
    {
      const int t = tid / SSM_COLS, cc = tid % SSM_COLS;
      const bool own = t < have && col0 + cc < A.dv;
      const float p = ldf(xbc + (size_t)(lo + r0 + (own ? t : 0)) * A.ld + x_at, own ? cc : 0);
      rx = own ? p : 0.f;
    }
    {
      const bool own = tid < C && tid < have;
      const float p = ldf(dtp + (size_t)(lo + r0 + (own ? tid : 0)) * A.ldt, A.dt_off + h);
      rdt = own ? p : 0.f;
    }
  };
  auto stage = [&]() {
#pragma unroll
    for (int j = 0; j < NBC; ++j) {
      const int idx = tid + 256 * j;
      sm[(idx / (2 * NP)) * ROWF + idx % (2 * NP)] = rbc[j];
    }
    sm[(tid / SSM_COLS) * ROWF + 2 * NP + tid % SSM_COLS] = rx;
    if (tid < C) {
      const float z = rdt + shift;
      const float dt = z > 20.f ? z : log1pf(expf(z));
      sm[tid * ROWF + 2 * NP + SSM_COLS] = dt;
      sm[tid * ROWF + 2 * NP + SSM_COLS + 1] = expf(-rate * dt);
    }
  };
  request(0);
  for (int r0 = 0; r0 < n; r0 += C) {
    __syncthreads();  // the chunk before has been read
    stage();
    __syncthreads();
    if (r0 + C < n) request(r0 + C);  // in flight while this chunk is worked through
    const int have = min(C, n - r0);
    // one token: the lane's rows of S move on and give its part of the read-out. No lane needs another's numbers for
    // the state (unlike the delta rule, whose write depends on a sum over the rows), so a full chunk's tokens are
    // worked through without a wait between them and their sums over the lanes are taken together afterwards; a
    // token's arithmetic is the same either way.
    auto token = [&](int t) {
      const float* row = sm + t * ROWF;
      const float dx = row[2 * NP + SSM_COLS] * row[2 * NP + cw], dA = row[2 * NP + SSM_COLS + 1];
      float y = 0.f;
#pragma unroll
      for (int e = 0; e < E; ++e) {
        S[e] = fmaf(dx, row[i0 + e], dA * S[e]);
        y = fmaf(S[e], row[NP + i0 + e], y);
      }
      return y;
    };
    if (!FEW && have == C) {
      float yp[C];
#pragma unroll
      for (int t = 0; t < C; ++t) yp[t] = token(t);
#pragma unroll
      for (int t = 0; t < C; ++t) yp[t] = ssm_row16_sum(yp[t]);
      float mine = yp[0];  // lane `part` of a column writes token `part`
#pragma unroll
      for (int t = 1; t < C; ++t) mine = part == t ? yp[t] : mine;
      if (col_on) A.out[(size_t)(lo + r0 + part) * A.ldo + (size_t)h * A.dv + col] = fmaf(skip, sm[part * ROWF + 2 * NP + cw], mine);
    } else {
      for (int t = 0; t < have; ++t) {
        const float y = ssm_row16_sum(token(t));
        if (part == 0 && col_on) A.out[(size_t)(lo + r0 + t) * A.ldo + (size_t)h * A.dv + col] = fmaf(skip, sm[t * ROWF + 2 * NP + cw], y);
      }
    }
  }
  if (wide) {
#pragma unroll
    for (int e = 0; e < E; e += 4)
      if (col_on && i0 + e < ns)
        *reinterpret_cast<float4*>(S_at + (size_t)col * ns + i0 + e) = make_float4(S[e], S[(e + 1) % E], S[(e + 2) % E], S[(e + 3) % E]);
  } else {
#pragma unroll
    for (int e = 0; e < E; ++e)
      if (col_on && i0 + e < ns) S_at[(size_t)col * ns + i0 + e] = S[e];
  }
}

extern "C" int jllm_ssm_scan(const void* xbc, int ld, const void* dt, int ldt, int dt_off, int dtype, const void* a_log,
                             const void* dt_bias, const void* skip, int w_dtype, float* state, float* out, int ldo,
                             const int* row_req, const int* state_slots, int n_rows, int n_requests, int heads, int groups,
                             int n, int dv, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (heads <= 0 || groups <= 0 || heads % groups || heads > 65535) JLLM_FAIL("ssm_scan: %d heads over %d groups", heads, groups);
  if (n <= 0 || n > SSM_PARTS * 16 || dv <= 0 || dv > SSM_COLS * 65535) JLLM_FAIL("ssm_scan: state size %d (1..%d are taken), value size %d", n, SSM_PARTS * 16, dv);
  if (n_requests <= 0 || n_requests > n_rows) JLLM_FAIL("ssm_scan: %d requests in %d rows", n_requests, n_rows);
  if (ld < heads * dv + 2 * groups * n || ldo < heads * dv || dt_off < 0 || ldt < dt_off + heads) JLLM_FAIL("ssm_scan: short rows");
  SsmArgs A{xbc, ld, dt, ldt, dt_off, a_log, dt_bias, skip, state, out, ldo, row_req, state_slots, n_rows, heads, groups, n, dv};
  dim3 grid(n_requests, heads, (dv + SSM_COLS - 1) / SSM_COLS);
  const int per_lane = (n + SSM_PARTS - 1) / SSM_PARTS;
  const bool few = n_rows <= 2 * n_requests;
#define SSM_LAUNCH(E)                                              \
  do {                                                             \
    if (few)                                                       \
      ssm_scan_kernel<T, TW, E, true><<<grid, 256, 0, stream>>>(A);  \
    else                                                           \
      ssm_scan_kernel<T, TW, E, false><<<grid, 256, 0, stream>>>(A); \
  } while (0)
  JLLM_DISPATCH_1(dtype, T, {
    JLLM_DISPATCH_1(w_dtype, TW, {
      if (per_lane <= 2)
        SSM_LAUNCH(2);
      else if (per_lane <= 4)
        SSM_LAUNCH(4);
      else if (per_lane <= 8)
        SSM_LAUNCH(8);
      else
        SSM_LAUNCH(16);
    })
  })
#undef SSM_LAUNCH
  JLLM_CHECK_LAUNCH("ssm_scan");
  return 0;
}

// ---------------------------------------------------------------------------------------------------------------------
// one workgroup per (row, group): t = y * silu(z) over the group's entries, out = t / sqrt(mean(t^2) + eps) * w
template <typename TZ, typename TW, typename TO>
__global__ __launch_bounds__(256) void gated_group_norm_kernel(const float* __restrict__ y, int ldy, const TZ* __restrict__ z,
                                                               int ldz, const TW* __restrict__ w, float eps, int per,
                                                               TO* __restrict__ out, int ldo) {
  __shared__ float red[4];
  const int r = blockIdx.x, g = blockIdx.y;
  const float* yr = y + (size_t)r * ldy + (size_t)g * per;
  const TZ* zr = z + (size_t)r * ldz + (size_t)g * per;
  float ss = 0.f;
  for (int i = threadIdx.x; i < per; i += 256) {
    const float zz = ldf(zr, i);
    const float t = yr[i] * (zz / (1.0f + expf(-zz)));
    ss = fmaf(t, t, ss);
  }
  ss = block_sum<4>(ss, red);
  const float s = norm_scale(ss, per, eps);
  for (int i = threadIdx.x; i < per; i += 256) {
    const float zz = ldf(zr, i);
    const float t = yr[i] * (zz / (1.0f + expf(-zz)));
    stf(out + (size_t)r * ldo, (size_t)g * per + i, (t * s) * ldf(w, (size_t)g * per + i));
  }
}

extern "C" int jllm_gated_group_norm(const float* y, int ldy, const void* z, int ldz, int z_dtype, const void* w, int w_dtype,
                                     float eps, int n_rows, int width, int groups, void* out, int out_dtype, int ldo,
                                     hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (width <= 0 || groups <= 0 || width % groups || groups > 65535) JLLM_FAIL("gated_group_norm: rows of %d in %d groups", width, groups);
  if (ldy < width || ldz < width || ldo < width) JLLM_FAIL("gated_group_norm: short rows");
  JLLM_DISPATCH_1(z_dtype, TZ, {
    JLLM_DISPATCH_1(w_dtype, TW, {
      JLLM_DISPATCH_1(out_dtype, TO, {
        gated_group_norm_kernel<TZ, TW, TO><<<dim3(n_rows, groups), 256, 0, stream>>>(y, ldy, (const TZ*)z, ldz, (const TW*)w, eps,
                                                                                     width / groups, (TO*)out, ldo);
      })
    })
  })
  JLLM_CHECK_LAUNCH("gated_group_norm");
  return 0;
}

// The attention of attention_dv.hip on the matrix cores, bf16 cache, for portions of prompts and single rows alike
// (flash style: no score matrix in memory, running maximum and sum in fp32, the output in fp32).
//
// Grid (query slot, tile). A tile is up to 128 consecutive rows of one request (4 waves x 32 rows); the caller lists the
// tiles as (request, first row, rows, position of the first row; a negative position means "the row's own entry of
// the positions array", for steps whose shape is fixed before their positions are known), the ones with the most keys
// first. Keys are walked in blocks of 64 aligned to absolute positions. Per block the workgroup stages the key slot's
// K [64][dk] and the value head's V [64][dv] in LDS as they lie in the cache (two buffers: the next block's loads
// are in flight while this one is multiplied); places outside the tile's visible range are stored as zeros and
// their table entries are never read. With kept first keys (keys before `keep_first` stay visible whatever the window)
// a tile's blocks are numbered: first the blocks of the kept keys that lie wholly before the window's first block, then
// the window's; a sink per head adds exp(sink) to the denominator where it is finished (here, or in the merge).
//
// Each wave computes the transposed scores S^T[key][row] = K Q^T (v_mfma_f32_32x32x16_bf16, A = K from LDS, B = Q
// in registers), so a lane owns one query row: maximum and sum are in-lane reductions plus one exchange between the
// half-waves. A cap on the scores (cap * tanh(s * scale / cap)) is applied to the accumulators before the softmax.
// The probabilities, rounded to bf16, are already laid out as the B operand of O^T[dim][row] += V^T P^T, whose A
// operand is read from V with the transposing LDS load (ds_read_b64_tr_b16). dk and dv are independent: dk in steps
// of 16 (the K loop), dv in blocks of 32 (the accumulators), both up to 256.
//
// Steps of single rows have few tiles with long chains of blocks: there gridDim.z workgroups share a tile's blocks
// (`per_split` blocks each, in order), each leaves its unnormalised sums, maximum and sum in a scratch array, and a
// second kernel merges them in the order of the splits. In such steps (`share` > 0) a workgroup also takes all query
// heads that read the same key slot and value head at once, one per lane of its first wave, in the place of the rows
// of a tile: the grid's x is then the key slot, and keys and values are read once for the whole group.
#include <math.h>

#include "common.h"
#include "mfma.h"

#define AT_KEYS 64

template <int DK16, int DB>
__global__ __launch_bounds__(256, (DK16 <= 8 && DB <= 4) ? 2 : 1) void attention_dv_tiles_kernel(
    const bf16_t* __restrict__ q, int ldq, float* __restrict__ out, int ldo, const bf16_t* __restrict__ kc,
    const bf16_t* __restrict__ vc, const int* __restrict__ block_table, int max_blocks, const int* __restrict__ tiles,
    const int* __restrict__ positions, int maps, int per_kv, int k_slots, int v_heads, int dv, int page_shift, int window,
    float scale, float softcap, float* __restrict__ partial, int per_split, int share, int q_slots, int keep_first,
    const float* __restrict__ sinks) {
  constexpr int DK = DK16 * 16;
  constexpr int DVP = DB * 32;
  constexpr int KLD = DK + 8;
  constexpr int VLD = DVP + 32;
  constexpr int KSZ = AT_KEYS * KLD;
  constexpr int VSZ = AT_KEYS * VLD;
  constexpr int KCH = (AT_KEYS * DK16 * 2 + 255) / 256;  // 16-byte pieces of K per thread and block
  constexpr int VPC = DVP / 8;                            // 16-byte pieces of a V row (the padded width)
  constexpr int VCH = (AT_KEYS * VPC + 255) / 256;
  extern __shared__ __align__(16) unsigned char smem_raw[];
  bf16_t* Ks = (bf16_t*)smem_raw;  // [2][KSZ]
  bf16_t* Vs = Ks + 2 * KSZ;       // [2][VSZ]
  const int* tile = tiles + (size_t)blockIdx.y * 4;
  const int req = tile[0], row0 = tile[1], nrows = tile[2];
  const int pos0 = tile[3] >= 0 ? tile[3] : positions[row0];
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int qi = lane & 31, half = lane >> 5;
  // share == 0: blockIdx.x is a query slot and the lanes of a wave are rows of the tile. share > 0 (tiles of one row):
  // blockIdx.x is a key slot and lane qi < share of the first wave is the qi-th query head that reads it
  const int vh = share ? (int)blockIdx.x / maps : (int)blockIdx.x / per_kv;
  const int ks_ = share ? (int)blockIdx.x : vh * maps + (int)blockIdx.x % maps;
  const int s = share ? (vh * share + min(qi, share - 1)) * maps + (int)blockIdx.x % maps : (int)blockIdx.x;
  const int wq = share ? 0 : wave * 32 + qi;                    // the lane's row within the tile
  const bool lane_on = share ? (wave == 0 && qi < share) : (wq < nrows);
  const int pos_q = pos0 + min(wq, nrows - 1);
  const int first_q = window > 0 ? max(0, pos_q + 1 - window) : 0;
  const int* tbl = block_table + (size_t)req * max_blocks;
  const int k_lo = window > 0 ? max(0, pos0 + 1 - window) : 0;
  const int k_hi = pos0 + nrows - 1;
  const int wave_lo_pos = pos0 + min(nrows - 1, wave * 32);
  const int wave_hi = pos0 + min(nrows - 1, wave * 32 + 31);
  const int wave_first = window > 0 ? max(0, wave_hi + 1 - window) : 0;
  const bool wave_on = share ? wave == 0 : wave * 32 < nrows;
  u32x4 qf[DK16];
  {
    const bf16_t* qr = q + (size_t)(row0 + min(wq, nrows - 1)) * ldq + (size_t)s * DK + half * 8;
#pragma unroll
    for (int i = 0; i < DK16; ++i) qf[i] = *(const u32x4*)(qr + i * 16);
  }
  // The blocks of a tile are numbered 0, 1, ...: first the blocks of the kept first keys that lie wholly before the
  // window's first block (keys before `kept` stay visible whatever the window), then the window's blocks.
  const int kept = window > 0 ? min(keep_first, k_lo) : 0;  // keys [0, kept) of the tile beside [k_lo, k_hi]
  const int win_first = (k_lo / AT_KEYS) * AT_KEYS;
  const int n_kept = min((kept + AT_KEYS - 1) / AT_KEYS, win_first / AT_KEYS);
  int it_first = 0;
  int n_blocks = n_kept + (k_hi - win_first) / AT_KEYS + 1;
  auto block_keys = [&](int it) { return it < n_kept ? it * AT_KEYS : win_first + (it - n_kept) * AT_KEYS; };
  if (partial) {  // this workgroup's share of the tile's blocks
    const int b0 = blockIdx.z * per_split;
    it_first = b0;
    n_blocks = min(per_split, n_blocks - b0);
    if (n_blocks <= 0) {  // nothing left for this split: it says so (the same for all threads: no barrier was met)
      if (lane_on && half == 0) {
        float* pr = partial + (((size_t)(row0 + wq) * q_slots + s) * gridDim.z + blockIdx.z) * (dv + 2);
        pr[dv] = -INFINITY;
        pr[dv + 1] = 0.f;
      }
      return;
    }
  }
  u32x4 kreg[KCH], vreg[VCH];
  int kpg[KCH], vpg[VCH];
  const int pmask = (1 << page_shift) - 1;
  auto load_pages = [&](int kt) {
#pragma unroll
    for (int j = 0; j < KCH; ++j) {
      const int c = tid + 256 * j;
      const int kabs = kt + c / (DK16 * 2);
      kpg[j] = (c < AT_KEYS * DK16 * 2 && (kabs >= k_lo || kabs < kept) && kabs <= k_hi) ? tbl[kabs >> page_shift] : -1;
    }
#pragma unroll
    for (int j = 0; j < VCH; ++j) {
      const int c = tid + 256 * j;
      const int kabs = kt + c / VPC;
      vpg[j] = (c < AT_KEYS * VPC && (c % VPC) * 8 < dv && (kabs >= k_lo || kabs < kept) && kabs <= k_hi) ? tbl[kabs >> page_shift] : -1;
    }
  };
  auto load_block = [&](int kt) {
#pragma unroll
    for (int j = 0; j < KCH; ++j) {
      const int c = tid + 256 * j;
      const int key = c / (DK16 * 2), pc = c % (DK16 * 2);
      kreg[j] = u32x4{0u, 0u, 0u, 0u};
      if (kpg[j] >= 0)
        kreg[j] = *(const u32x4*)(kc + ((((size_t)kpg[j] * k_slots + ks_) << page_shift) + ((kt + key) & pmask)) * DK + pc * 8);
    }
#pragma unroll
    for (int j = 0; j < VCH; ++j) {
      const int c = tid + 256 * j;
      const int key = c / VPC, pc = c % VPC;
      vreg[j] = u32x4{0u, 0u, 0u, 0u};
      if (vpg[j] >= 0)
        vreg[j] = *(const u32x4*)(vc + ((((size_t)vpg[j] * v_heads + vh) << page_shift) + ((kt + key) & pmask)) * dv + pc * 8);
    }
  };
  auto store_block = [&](int buf) {
    bf16_t* kd = Ks + buf * KSZ;
    bf16_t* vd = Vs + buf * VSZ;
#pragma unroll
    for (int j = 0; j < KCH; ++j) {
      const int c = tid + 256 * j;
      if (c >= AT_KEYS * DK16 * 2) continue;
      *(u32x4*)(kd + (size_t)(c / (DK16 * 2)) * KLD + (c % (DK16 * 2)) * 8) = kreg[j];
    }
#pragma unroll
    for (int j = 0; j < VCH; ++j) {
      const int c = tid + 256 * j;
      if (c >= AT_KEYS * VPC) continue;
      *(u32x4*)(vd + (size_t)(c / VPC) * VLD + (c % VPC) * 8) = vreg[j];
    }
  };
  // what this lane names in a transposing load of V: key 4 half + (lane % 16) / 4, dims 16 ((lane / 16) % 2) + 4 (lane % 4)
  const int v_lane = (half * 4 + ((lane & 15) >> 2)) * VLD + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
  floatx16 o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) o[db][e] = 0.f;
  float m = -INFINITY, l = 0.f;
  const float log2e = 1.4426950408889634f;
  const float sl = softcap > 0.f ? log2e : scale * log2e;  // capped scores are final; raw ones are scaled in the exponent
  const float cap_in = softcap > 0.f ? 2.0f * log2e * scale / softcap : 0.f;
  // beyond a tile's last block the block numbers name keys past k_hi, whose table entries are never read
  load_pages(block_keys(it_first));
  load_block(block_keys(it_first));
  load_pages(block_keys(it_first + 1));
  store_block(0);
  __syncthreads();
  int buf = 0;
  for (int it = 0; it < n_blocks; ++it, buf ^= 1) {
    const int kt = block_keys(it_first + it);
    const bool more = it + 1 < n_blocks;
    if (more) {
      load_block(block_keys(it_first + it + 1));
      load_pages(block_keys(it_first + it + 2));
    }
    if (wave_on && kt <= wave_hi) {
      const bf16_t* Kb = Ks + buf * KSZ;
      const bf16_t* Vb = Vs + buf * VSZ + v_lane;
      floatx16 sc[2];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
        for (int e = 0; e < 16; ++e) sc[kb][e] = 0.f;
        const bf16_t* kr = Kb + (size_t)(kb * 32 + qi) * KLD + half * 8;
#pragma unroll
        for (int i = 0; i < DK16; ++i) sc[kb] = mfma32(*(const u32x4*)(kr + i * 16), qf[i], sc[kb]);
      }
      if (softcap > 0.f) {  // cap * tanh(x), tanh(x) = 1 - 2 / (1 + exp(2x))
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int e = 0; e < 16; ++e)
            sc[kb][e] = softcap * (1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(sc[kb][e] * cap_in)));
      }
      const bool all_visible = kt + AT_KEYS - 1 <= wave_lo_pos && (kt >= wave_first || kt + AT_KEYS <= kept);
      if (!all_visible) {
        const int key0 = kt + half * 4;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            const int key = key0 + kb * 32 + 8 * (e >> 2) + (e & 3);
            sc[kb][e] = ((key >= first_q || key < keep_first) && key <= pos_q) ? sc[kb][e] : -INFINITY;
          }
      }
      // the maximum of the scores as they enter the exponent (a negative scale turns the order round)
      float mx = -INFINITY;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int e = 0; e < 16; ++e) mx = fmaxf(mx, sc[kb][e] * sl);
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float m_new = (mx > m + 8.0f) ? mx : m;  // moves only when it grows by more than 2^8
      u32x4 pb[2][2];
      if (m_new == -INFINITY) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int st = 0; st < 2; ++st) pb[kb][st] = u32x4{0u, 0u, 0u, 0u};
      } else {
        float rs = 0.f;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
          float p[16];
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            p[e] = __builtin_amdgcn_exp2f(fmaf(sc[kb][e], sl, -m_new));
            rs += p[e];
          }
#pragma unroll
          for (int st = 0; st < 2; ++st)
            pb[kb][st] = u32x4{pack_bf16(p[8 * st], p[8 * st + 1]), pack_bf16(p[8 * st + 2], p[8 * st + 3]),
                               pack_bf16(p[8 * st + 4], p[8 * st + 5]), pack_bf16(p[8 * st + 6], p[8 * st + 7])};
        }
        rs += __shfl_xor(rs, 32, 64);
        if (m_new != m) {
          const float alpha = __builtin_amdgcn_exp2f(m - m_new);
          l *= alpha;
#pragma unroll
          for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int e = 0; e < 16; ++e) o[db][e] *= alpha;
          m = m_new;
        }
        l += rs;
      }
#pragma unroll
      for (int db = 0; db < DB; ++db) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int st = 0; st < 2; ++st) {
            const int k0 = kb * 32 + 16 * st;
            const u32x2 lo = lds_read_tr16(Vb + k0 * VLD + db * 32);
            const u32x2 hi = lds_read_tr16(Vb + (k0 + 8) * VLD + db * 32);
            o[db] = mfma32(u32x4{lo.x, lo.y, hi.x, hi.y}, pb[kb][st], o[db]);
          }
      }
    }
    if (more) store_block(buf ^ 1);
    __syncthreads();
  }
  if (!wave_on || !lane_on) return;
  if (partial) {
    float* pr = partial + (((size_t)(row0 + wq) * q_slots + s) * gridDim.z + blockIdx.z) * (dv + 2);
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int d = db * 32 + 8 * (e >> 2) + half * 4 + (e & 3);
        if (d < dv) pr[d] = o[db][e];
      }
    if (half == 0) {
      pr[dv] = m;
      pr[dv + 1] = l;
    }
    return;
  }
  // a sink is one more term of the denominator, exp(sink), with no value; m is an exponent of two
  if (sinks) l += __builtin_amdgcn_exp2f(sinks[s / maps] * log2e - m);
  const float inv = 1.0f / l;
  float* orow = out + (size_t)(row0 + wq) * ldo + (size_t)s * dv;
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int e4 = 0; e4 < 4; ++e4) {
      const int d = db * 32 + 8 * e4 + half * 4;
      if (d < dv) *(float4*)(orow + d) = float4{o[db][4 * e4] * inv, o[db][4 * e4 + 1] * inv, o[db][4 * e4 + 2] * inv, o[db][4 * e4 + 3] * inv};
    }
}

// partial [rows][q_slots][splits][dv + 2]: unnormalised sums, then the maximum (as an exponent of two) and the sum.
// Lane z holds split z's maximum and sum (at most 64 splits), so the weights of all splits are known after two wave
// reductions and the sums' loads are independent of each other.
__global__ __launch_bounds__(64) void attention_dv_merge_kernel(const float* __restrict__ partial, int splits, int dv,
                                                                float* __restrict__ out, int ldo, int maps,
                                                                const float* __restrict__ sinks) {
  const int t = blockIdx.x, s = blockIdx.y, lane = threadIdx.x;
  const float* pr = partial + ((size_t)t * gridDim.y + s) * splits * (dv + 2);
  const float mz = lane < splits ? pr[(size_t)lane * (dv + 2) + dv] : -INFINITY;
  const float lz = lane < splits ? pr[(size_t)lane * (dv + 2) + dv + 1] : 0.f;
  const float mx = wave_max(mz);
  const float wz = mz == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mz - mx);
  const float sink_term = sinks ? __builtin_amdgcn_exp2f(sinks[s / maps] * 1.4426950408889634f - mx) : 0.f;
  const float inv = 1.0f / (wave_sum(lz * wz) + sink_term);
  for (int d = lane; d < dv; d += 64) {
    float acc = 0.f;
#pragma unroll 4
    for (int z = 0; z < splits; ++z) {
      const float w = __shfl(wz, z, 64);
      const float v = pr[(size_t)z * (dv + 2) + d];
      acc = w != 0.f ? fmaf(v, w, acc) : acc;  // a split without keys left its sums unwritten
    }
    out[(size_t)t * ldo + (size_t)s * dv + d] = acc * inv;
  }
}

template <int DK16, int DB>
static int launch_tiles(dim3 grid, hipStream_t stream, const bf16_t* q, int ldq, float* out, int ldo, const bf16_t* kc,
                        const bf16_t* vc, const int* block_table, int max_blocks, const int* tiles, const int* positions, int maps,
                        int per_kv, int k_slots, int v_heads, int dv, int page_shift, int window, float scale, float softcap,
                        float* partial, int per_split, int share, int q_slots, int keep_first, const float* sinks) {
  const size_t smem = (size_t)2 * AT_KEYS * ((DK16 * 16 + 8) + (DB * 32 + 32)) * sizeof(bf16_t);
  static bool raised = false;
  if (smem > 64 * 1024 && !raised) {
    if (hipFuncSetAttribute((const void*)attention_dv_tiles_kernel<DK16, DB>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess)
      return -1;
    raised = true;
  }
  attention_dv_tiles_kernel<DK16, DB><<<grid, 256, smem, stream>>>(q, ldq, out, ldo, kc, vc, block_table, max_blocks, tiles, positions,
                                                                 maps, per_kv, k_slots, v_heads, dv, page_shift, window, scale, softcap,
                                                                 partial, per_split, share, q_slots, keep_first, sinks);
  return 0;
}

// Returns 1 (declined) for sizes it does not take: dk a multiple of 16 up to 256, dv a multiple of 8 up to 256, bf16.
// `splits` > 1 (tiles of single rows only): the workgroups of a tile take `per_split` key blocks each and `partial`
// (fp32, rows x slots x splits x (dv + 2)) carries their results to the merge (a kernel of its own here, or, with
// `defer_merge`, the prologue of the kernel that finishes the heads).
extern "C" int jllm_attention_dv_bf16(const void* q, int ldq, float* out, int ldo, const void* kcache, const void* vcache,
                                      const int* block_table, int max_blocks, const int* tiles, int n_tiles,
                                      const int* positions, int heads, int kv_heads, int maps, int dk, int dv, int page_size,
                                      int window, float scale, float softcap, int splits, int per_split, float* partial,
                                      int n_rows, int defer_merge, int keep_first, const float* sinks, hipStream_t stream) {
  if (n_tiles <= 0) return 0;
  if (heads <= 0 || kv_heads <= 0 || heads % kv_heads != 0 || maps <= 0) JLLM_FAIL("attention: %d query heads over %d kv heads with %d maps", heads, kv_heads, maps);
  if ((dk & 15) || dk < 16 || dk > 256 || (dv & 7) || dv < 8 || dv > 256) return 1;
  if (!(scale > 0.f) || softcap < 0.f || keep_first < 0) return 1;  // the maximum is taken before the scale's sign could matter
  if ((ldq & 7) || (ldo & 3) || ((uintptr_t)q & 15) || ((uintptr_t)out & 15) || ((uintptr_t)kcache & 15) || ((uintptr_t)vcache & 15)) return 1;
  if (page_size <= 0 || (page_size & (page_size - 1)) || n_tiles > 65535 || heads * maps > 65535) return 1;
  int page_shift = 0;
  while ((1 << page_shift) < page_size) ++page_shift;
  const int q_slots = heads * maps, per_kv = maps * (heads / kv_heads);
  if (splits > 1 && (!partial || per_split <= 0 || n_rows != n_tiles || splits > 64)) JLLM_FAIL("attention: %d splits of %d blocks over %d tiles of %d rows", splits, per_split, n_tiles, n_rows);
  if (splits <= 1) partial = nullptr;
  // tiles of one row: the heads of a key slot share a workgroup (up to the 32 lanes that hold a tile's rows)
  const int share = (n_rows == n_tiles && heads / kv_heads > 1 && heads / kv_heads <= 32) ? heads / kv_heads : 0;
  dim3 grid(share ? kv_heads * maps : q_slots, n_tiles, partial ? splits : 1);
  const int db = (dv + 31) / 32;
  int rc = 1;
#define AT_ARGS grid, stream, (const bf16_t*)q, ldq, out, ldo, (const bf16_t*)kcache, (const bf16_t*)vcache, block_table, max_blocks, \
                tiles, positions, maps, per_kv, kv_heads * maps, kv_heads, dv, page_shift, window, scale, softcap, partial, per_split, \
                share, q_slots, keep_first, sinks
#define AT_DB(N)                                  \
  switch (db) {                                   \
    case 1: rc = launch_tiles<N, 1>(AT_ARGS); break; \
    case 2: rc = launch_tiles<N, 2>(AT_ARGS); break; \
    case 3: rc = launch_tiles<N, 3>(AT_ARGS); break; \
    case 4: rc = launch_tiles<N, 4>(AT_ARGS); break; \
    case 8: rc = launch_tiles<N, 8>(AT_ARGS); break; \
    default: return 1;                            \
  }
  switch (dk / 16) {
    case 1: AT_DB(1) break;
    case 2: AT_DB(2) break;
    case 3: AT_DB(3) break;
    case 4: AT_DB(4) break;
    case 6: AT_DB(6) break;
    case 8: AT_DB(8) break;
    case 16: AT_DB(16) break;
    default: return 1;
  }
#undef AT_DB
#undef AT_ARGS
  if (rc < 0) JLLM_FAIL("attention: cannot reserve LDS");
  // `defer_merge`: the caller's next kernel reads the splits itself (heads_finish_split in attention_dv.hip)
  if (partial && !defer_merge) attention_dv_merge_kernel<<<dim3(n_rows, q_slots), 64, 0, stream>>>(partial, splits, dv, out, ldo, maps, sinks);
  JLLM_CHECK_LAUNCH("attention_dv_bf16");
  return 0;
}

// Sliding-window softmax attention over a paged cache that also sees block means of the keys and
// values behind the window, with capped scores, sink logits and mixing of the heads' weights.
//
//   pool_update        for a token at the last position of a block of `pool`: the mean of the block's
//                      cached key / value rows goes to entry position / pool of the mean caches
//   pooled_attention   query at position p sees single keys max(0, p - window + 1) <= j <= p and the
//                      means of blocks b < floor((p - window + 1) / pool);  s = cap tanh(q . k scale / cap);
//                      p_j = exp(s_j) / (exp(sink_h) + sum exp(s_j')) over both kinds of keys;
//                      out[t, h, g] = sum_j p_j v_(g, j) for every value head g (all_values) or the own one
//   mix_heads          out[t, h] = post * sum_g talk[h, g] o[t, g, value head of h]
//
// Scores, softmax, means and sums are fp32 for both element types.  The (token, head) pairs of a
// sequence that share a key head are the rows of one tile problem against key / value tiles staged
// once in LDS; the tiles of the means and of the single keys each start at multiples of the tile
// size counted from entry 0 of the sequence, so a position's sums run in the same order however its
// prompt was cut and whatever else the step holds.
#include <hip/hip_runtime.h>

#include <cmath>

#include "mix_common.h"

using namespace pkm;

namespace {

// one workgroup per (token, key head): thread c sums column c of the block's rows in position order
template <typename T>
__global__ void __launch_bounds__(256)
pool_update_kernel(const T* __restrict__ k_cache, const T* __restrict__ v_cache, T* __restrict__ kp_cache,
                   T* __restrict__ vp_cache, const int* __restrict__ positions, const int* __restrict__ slot_mapping,
                   const int* __restrict__ token_seq, const int* __restrict__ block_tables, int64_t bt_stride, int G, int D,
                   int V, int bs, int pool) {
  const int t = blockIdx.x, g = blockIdx.y;
  const int pos = positions[t];
  if (pos < 0 || (pos + 1) % pool != 0 || (slot_mapping && slot_mapping[t] < 0)) return;
  const int* bt = block_tables + static_cast<int64_t>(token_seq[t]) * bt_stride;
  const int b = pos / pool;
  const int64_t dst = (static_cast<int64_t>(bt[b / bs]) * G + g) * bs + b % bs;
  const float inv = 1.f / static_cast<float>(pool);
  for (int c = threadIdx.x; c < D + V; c += 256) {
    const bool key = c < D;
    const T* src = key ? k_cache : v_cache;
    const int w = key ? D : V, cc = key ? c : c - D;
    float acc = 0.f;
    for (int j = pos - pool + 1; j <= pos; ++j)
      acc += ld<T>(src + ((static_cast<int64_t>(bt[j / bs]) * G + g) * bs + j % bs) * w + cc);
    st<T>((key ? kp_cache : vp_cache) + dst * w + cc, acc * inv);
  }
}

constexpr int kBQ = 16;        // (token, head) rows per workgroup
constexpr int kThreads = 256;  // 16 rows x 16 lanes

struct PooledArgs {
  float* out;  // [T, H, VG, V]
  const void* q;  // [T, H, D]
  const void *k_cache, *v_cache, *kp_cache, *vp_cache;  // [blocks, G, bs, D | V]
  const int* block_tables;
  int64_t bt_stride;
  const int* cu_q;
  const int* context_lens;
  const float* sink;  // [H] logits or null
  int n_seqs, H, G, D, V, bs, BK;
  float scale, softcap;
  int window, pool, all_values;
  // few rows (decoded tokens): the key tiles are dealt to n_parts workgroups per row tile, which leave
  // (max, sum, unnormalised sums) in the workspace for pooled_merge_kernel (the sink joins there)
  int n_parts;
  float* ws_acc;  // [T * H, n_parts, VW]
  float* ws_ml;   // [T * H, n_parts, 2]
};

// 16 bytes of a cache row as floats
template <typename T>
struct Chunk;
template <>
struct Chunk<float> {
  static constexpr int N = 4;
  __device__ static __forceinline__ void load(const float* p, float* f) {
    const float4 v = *reinterpret_cast<const float4*>(p);
    f[0] = v.x, f[1] = v.y, f[2] = v.z, f[3] = v.w;
  }
};
template <>
struct Chunk<bf16_t> {
  static constexpr int N = 8;
  __device__ static __forceinline__ void load(const bf16_t* p, float* f) {
    const uint4 v = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __uint_as_float(w[i] << 16);
      f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
};

// rows [j0, j0 + BK) x width columns of a paged cache into an LDS tile with row stride `stride`:
// 16-byte loads when the width allows (all loads of a pass are issued before the first LDS store)
template <typename T>
__device__ __forceinline__ void stage_tile(float* tile, int stride, const T* cache, const int* bt, int bs, int heads,
                                           int head0, int n_heads, int width, int k0, int nk, int BK, int tid) {
  constexpr int N = Chunk<T>::N;
  const int W = n_heads * width;  // columns of the tile: n_heads heads side by side
  if (width % N == 0) {
    const int per = W / N, units = BK * per;
    constexpr int kPass = 4;
    for (int u0 = 0; u0 < units; u0 += kPass * kThreads) {
      float f[kPass][N];
#pragma unroll
      for (int p = 0; p < kPass; ++p) {
        const int u = u0 + p * kThreads + tid;
        const int j = u / per, c = (u - j * per) * N;
        if (u < units && j < nk) {
          const int key = k0 + j, g = c / width, cc = c - g * width;
          Chunk<T>::load(cache + ((static_cast<int64_t>(bt[key / bs]) * heads + head0 + g) * bs + key % bs) * width + cc, f[p]);
        } else {
#pragma unroll
          for (int i = 0; i < N; ++i) f[p][i] = 0.f;
        }
      }
#pragma unroll
      for (int p = 0; p < kPass; ++p) {
        const int u = u0 + p * kThreads + tid;
        if (u < units) {
          const int j = u / per, c = (u - j * per) * N;
#pragma unroll
          for (int i = 0; i < N; ++i) tile[j * stride + c + i] = f[p][i];
        }
      }
    }
    return;
  }
  for (int e = tid; e < BK * W; e += kThreads) {
    const int j = e / W, c = e - j * W;
    float v = 0.f;
    if (j < nk) {
      const int key = k0 + j, g = c / width, cc = c - g * width;
      v = ld<T>(cache + ((static_cast<int64_t>(bt[key / bs]) * heads + head0 + g) * bs + key % bs) * width + cc);
    }
    tile[j * stride + c] = v;
  }
}

__device__ __forceinline__ int blocks_seen(int pos, int window, int pool) {
  if (window <= 0 || pool <= 0) return 0;
  const int n = pos - window + 1;
  return n >= pool ? n / pool : 0;
}

// NV: output accumulators per thread and row = ceil(value columns / 64)
template <typename T, int NV>
__global__ void __launch_bounds__(kThreads) pooled_attention_kernel(PooledArgs a) {
  extern __shared__ float smem[];
  const int H = a.H, G = a.G, D = a.D, V = a.V, BK = a.BK, bs = a.bs;
  const int R = H / G;
  const int kh = blockIdx.y;
  const int VG = a.all_values ? G : 1;
  const int VW = VG * V;  // value columns staged per key
  int s = 0, tile = blockIdx.x;
  for (; s < a.n_seqs; ++s) {
    const int rows = (a.cu_q[s + 1] - a.cu_q[s]) * R;
    const int nt = (rows + kBQ - 1) / kBQ;
    if (tile < nt) break;
    tile -= nt;
  }
  if (s >= a.n_seqs) return;
  const int q0 = a.cu_q[s], qlen = a.cu_q[s + 1] - q0, ctx = a.context_lens[s];
  const int n_rows = qlen * R;
  const int row0 = tile * kBQ;
  const int DS = D + 1, VS = VW + 1;  // odd row strides: conflict-free column walks
  float* qs = smem;             // [kBQ][DS]
  float* ks = qs + kBQ * DS;    // [BK][DS]
  float* vs = ks + BK * DS;     // [BK][VS]
  float* ps = vs + BK * VS;     // [kBQ][BK]
  float* m_s = ps + kBQ * BK;   // [kBQ] running max
  float* l_s = m_s + kBQ;       // [kBQ] running sum
  float* r_s = l_s + kBQ;       // [kBQ] the current tile's rescale of each row's sums
  const int tid = threadIdx.x;
  const int qi = tid >> 4, kg = tid & 15;
  const int* bt = a.block_tables + static_cast<int64_t>(s) * a.bt_stride;

  for (int e = tid; e < kBQ * D; e += kThreads) {
    const int r = e / D, c = e - r * D;
    const int row = row0 + r;
    float v = 0.f;
    if (row < n_rows) {
      const int tl = row / R, h = kh * R + row - tl * R;
      v = ld<T>(static_cast<const T*>(a.q) + (static_cast<int64_t>(q0 + tl) * H + h) * D + c);
    }
    qs[r * DS + c] = v;
  }
  const int my_row = row0 + qi;
  const bool live = my_row < n_rows;
  const int my_tl = live ? my_row / R : 0;
  const int my_h = kh * R + (live ? my_row - my_tl * R : 0);
  const int my_pos = live ? ctx - qlen + my_tl : -1;
  const int my_lo = (live && a.window > 0) ? max(0, my_pos - a.window + 1) : 0;
  const int my_blocks = live ? blocks_seen(my_pos, a.window, a.pool) : 0;
  if (tid < kBQ) {
    const int row = row0 + tid;
    const int h = kh * R + (row < n_rows ? row % R : 0);
    const bool sink_here = a.sink && a.n_parts <= 1;
    m_s[tid] = sink_here ? a.sink[h] : -INFINITY;  // the sink is a key without a value
    l_s[tid] = sink_here ? 1.f : 0.f;
  }
  const int first_pos = ctx - qlen + row0 / R;
  const int last_pos = ctx - qlen + (min(row0 + kBQ, n_rows) - 1) / R;
  // value sums: thread (rg, cl) owns rows 4 rg .. 4 rg + 3 and columns cl + 64 i, so a value read from LDS
  // meets four rows; row groups past the tile's rows (decoded tokens: R rows) sit the products out
  const int rg = tid >> 6, cl = tid & 63;
  const bool pv_live = row0 + 4 * rg < n_rows;
  float acc[4][NV];
#pragma unroll
  for (int r = 0; r < 4; ++r)
#pragma unroll
    for (int i = 0; i < NV; ++i) acc[r][i] = 0.f;
  __syncthreads();

  // part 0: the block means (entries [0, blocks seen by the tile's last row)); part 1: single keys
  int tile_no = 0;
  for (int part = 0; part < 2; ++part) {
    const T* kc = static_cast<const T*>(part ? a.k_cache : a.kp_cache);
    const T* vc = static_cast<const T*>(part ? a.v_cache : a.vp_cache);
    int k_begin, k_end;
    if (part == 0) {
      k_begin = 0;
      k_end = last_pos >= 0 ? blocks_seen(last_pos, a.window, a.pool) : 0;
    } else {
      k_end = last_pos + 1;
      k_begin = (first_pos >= 0 && a.window > 0) ? max(0, first_pos - a.window + 1) / BK * BK : 0;
    }
    for (int k0 = k_begin; k0 < k_end; k0 += BK) {
      if (a.n_parts > 1 && (tile_no++) % a.n_parts != static_cast<int>(blockIdx.z)) continue;
      const int nk = min(BK, k_end - k0);
      stage_tile<T>(ks, DS, kc, bt, bs, G, kh, 1, D, k0, nk, BK, tid);
      stage_tile<T>(vs, VS, vc, bt, bs, G, a.all_values ? 0 : kh, VG, V, k0, nk, BK, tid);
      __syncthreads();
      float tmax = -INFINITY;
      for (int j = kg; j < BK; j += 16) {
        const int key = k0 + j;
        const bool seen = j < nk && live && (part == 0 ? key < my_blocks : (key <= my_pos && key >= my_lo));
        float d = -INFINITY;
        if (seen) {
          d = 0.f;
          const float* qr = qs + qi * DS;
          const float* kr = ks + j * DS;
          for (int c = 0; c < D; ++c) d += qr[c] * kr[c];
          d *= a.scale;
          if (a.softcap > 0.f) d = a.softcap * tanhf(d / a.softcap);
        }
        ps[qi * BK + j] = d;
        tmax = fmaxf(tmax, d);
      }
#pragma unroll
      for (int o = 8; o > 0; o >>= 1) tmax = fmaxf(tmax, __shfl_xor(tmax, o, 64));
      const float m_old = m_s[qi];
      const float m_new = fmaxf(m_old, tmax);
      float tsum = 0.f;
      for (int j = kg; j < BK; j += 16) {
        const float sc = ps[qi * BK + j];
        const float p = (m_new == -INFINITY || sc == -INFINITY) ? 0.f : expf(sc - m_new);
        ps[qi * BK + j] = p;
        tsum += p;
      }
#pragma unroll
      for (int o = 8; o > 0; o >>= 1) tsum += __shfl_xor(tsum, o, 64);
      const float resc = (m_old == -INFINITY) ? 0.f : expf(m_old - m_new);
      if (kg == 0) r_s[qi] = resc;
      __syncthreads();  // every lane of the row has read m_old and its own scores
      if (kg == 0) {
        m_s[qi] = m_new;
        l_s[qi] = l_s[qi] * resc + tsum;
      }
      if (pv_live) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float rs = r_s[4 * rg + r];
#pragma unroll
          for (int i = 0; i < NV; ++i) acc[r][i] *= rs;
        }
        for (int j = 0; j < nk; ++j) {
          float p[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) p[r] = ps[(4 * rg + r) * BK + j];
          const float* vr = vs + j * VS + cl;
#pragma unroll
          for (int i = 0; i < NV; ++i) {
            if (cl + 64 * i < VW) {
              const float v = vr[64 * i];
#pragma unroll
              for (int r = 0; r < 4; ++r) acc[r][i] += p[r] * v;
            }
          }
        }
      }
      __syncthreads();
    }
  }
  if (!pv_live) return;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int row = row0 + 4 * rg + r;
    if (row >= n_rows) break;
    const int tl = row / R, h = kh * R + row - tl * R;
    const float l = l_s[4 * rg + r];
    if (a.n_parts > 1) {
      const int64_t slot = (static_cast<int64_t>(q0 + tl) * H + h) * a.n_parts + blockIdx.z;
      float* dst = a.ws_acc + slot * VW;
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int c = cl + 64 * i;
        if (c < VW) dst[c] = acc[r][i];
      }
      if (cl == 0) {
        a.ws_ml[2 * slot] = m_s[4 * rg + r];
        a.ws_ml[2 * slot + 1] = l;
      }
    } else {
      const float inv = l > 0.f ? 1.f / l : 0.f;
      float* dst = a.out + (static_cast<int64_t>(q0 + tl) * H + h) * VW;
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int c = cl + 64 * i;
        if (c < VW) dst[c] = acc[r][i] * inv;
      }
    }
  }
}

// ---- bf16 on the matrix cores -------------------------------------------------------------------
// The same tile problem (16 (token, head) rows of one key head against 32-key tiles, block means first) with
// both products on mfma_f32_16x16x32_bf16.  Lane (g, n) = (lane / 16, lane % 16) supplies A[row n][k 8g..8g+7]
// and B[k 8g..8g+7][column n] and holds C[rows 4g..4g+3][column n].
//   S [rows x keys]  = Q [rows x D] . K^T       A = query rows, B = key rows, both 16-byte reads of bf16 LDS tiles
//   O [rows x cols] += P [rows x keys] . V      A = the softmax weights as two bf16 parts (leading part and
//                                               remainder, two instructions), B = a value column's 8 keys
// Tiles are staged as they lie in the cache (16-byte copies, no conversion).  Wave w takes the 16-key blocks
// w, w + 4, .. of the first product and the 16-column blocks w, w + 4, .. of the second; cap, band, sink and the
// running maximum / sum stay with the 16 x 16 thread layout of the FMA kernel.
template <int NV>
__global__ void __launch_bounds__(kThreads) pooled_attention_mfma_kernel(PooledArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  const int H = a.H, G = a.G, D = a.D, V = a.V, BK = a.BK, bs = a.bs;
  const int R = H / G;
  const int kh = blockIdx.y;
  const int VG = a.all_values ? G : 1;
  const int VW = VG * V;
  int s = 0, tile = blockIdx.x;
  for (; s < a.n_seqs; ++s) {
    const int rows = (a.cu_q[s + 1] - a.cu_q[s]) * R;
    const int nt = (rows + kBQ - 1) / kBQ;
    if (tile < nt) break;
    tile -= nt;
  }
  if (s >= a.n_seqs) return;
  const int q0 = a.cu_q[s], qlen = a.cu_q[s + 1] - q0, ctx = a.context_lens[s];
  const int n_rows = qlen * R;
  const int row0 = tile * kBQ;
  const int DSH = D + 8, VSH = VW + 8, PSH = BK + 8;  // bf16 row strides: rows stay 16-byte aligned, banks shift
  bf16_t* qs = reinterpret_cast<bf16_t*>(smem_raw);  // [kBQ][DSH]
  bf16_t* ks = qs + kBQ * DSH;                       // [BK][DSH]
  bf16_t* vs = ks + BK * DSH;                        // [BK][VSH]
  bf16_t* pb = vs + BK * VSH;                        // [2][kBQ][PSH] softmax weights as bf16: leading part, remainder
  bf16_t* pb2 = pb + kBQ * PSH;
  float* ps = reinterpret_cast<float*>(pb2 + kBQ * PSH);  // [kBQ][BK] scores, then weights
  float* m_s = ps + kBQ * BK;
  float* l_s = m_s + kBQ;
  float* r_s = l_s + kBQ;
  const int tid = threadIdx.x;
  const int qi = tid >> 4, kg = tid & 15;
  const int lane = tid & 63, w = tid >> 6, g4 = lane >> 4, n = lane & 15;
  const int* bt = a.block_tables + static_cast<int64_t>(s) * a.bt_stride;
  const uint4 zero4 = uint4{0u, 0u, 0u, 0u};

  for (int u = tid; u < kBQ * (D / 8); u += kThreads) {
    const int r = u / (D / 8), c = (u - r * (D / 8)) * 8;
    const int row = row0 + r;
    uint4 v = zero4;
    if (row < n_rows) {
      const int tl = row / R, h = kh * R + row - tl * R;
      v = *reinterpret_cast<const uint4*>(static_cast<const bf16_t*>(a.q) + (static_cast<int64_t>(q0 + tl) * H + h) * D + c);
    }
    *reinterpret_cast<uint4*>(qs + r * DSH + c) = v;
  }
  const int my_row = row0 + qi;
  const bool live = my_row < n_rows;
  const int my_tl = live ? my_row / R : 0;
  const int my_pos = live ? ctx - qlen + my_tl : -1;
  const int my_lo = (live && a.window > 0) ? max(0, my_pos - a.window + 1) : 0;
  const int my_blocks = live ? blocks_seen(my_pos, a.window, a.pool) : 0;
  if (tid < kBQ) {
    const int row = row0 + tid;
    const int h = kh * R + (row < n_rows ? row % R : 0);
    const bool sink_here = a.sink && a.n_parts <= 1;
    m_s[tid] = sink_here ? a.sink[h] : -INFINITY;
    l_s[tid] = sink_here ? 1.f : 0.f;
  }
  const int first_pos = ctx - qlen + row0 / R;
  const int last_pos = ctx - qlen + (min(row0 + kBQ, n_rows) - 1) / R;
  pk::f32x4 acc[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) acc[i] = pk::f32x4{0.f, 0.f, 0.f, 0.f};
  __syncthreads();

  int tile_no = 0;
  for (int part = 0; part < 2; ++part) {
    const bf16_t* kc = static_cast<const bf16_t*>(part ? a.k_cache : a.kp_cache);
    const bf16_t* vc = static_cast<const bf16_t*>(part ? a.v_cache : a.vp_cache);
    int k_begin, k_end;
    if (part == 0) {
      k_begin = 0;
      k_end = last_pos >= 0 ? blocks_seen(last_pos, a.window, a.pool) : 0;
    } else {
      k_end = last_pos + 1;
      k_begin = (first_pos >= 0 && a.window > 0) ? max(0, first_pos - a.window + 1) / BK * BK : 0;
    }
    for (int k0 = k_begin; k0 < k_end; k0 += BK) {
      if (a.n_parts > 1 && (tile_no++) % a.n_parts != static_cast<int>(blockIdx.z)) continue;
      const int nk = min(BK, k_end - k0);
      {  // key rows, then the value rows of the staged value heads: 16-byte copies, four per thread and pass
        const int kper = D / 8, vper = VW / 8;
        const int units = BK * (kper + vper);
        for (int u0 = 0; u0 < units; u0 += 4 * kThreads) {
          uint4 v[4];
#pragma unroll
          for (int p = 0; p < 4; ++p) {
            const int u = u0 + p * kThreads + tid;
            v[p] = zero4;
            if (u < BK * kper) {
              const int j = u / kper, c = (u - j * kper) * 8;
              if (j < nk) {
                const int key = k0 + j;
                v[p] = *reinterpret_cast<const uint4*>(kc + ((static_cast<int64_t>(bt[key / bs]) * G + kh) * bs + key % bs) * D + c);
              }
            } else if (u < units) {
              const int u2 = u - BK * kper;
              const int j = u2 / vper, c = (u2 - j * vper) * 8;
              if (j < nk) {
                const int key = k0 + j;
                const int g = a.all_values ? c / V : kh, cc = a.all_values ? c - g * V : c;
                v[p] = *reinterpret_cast<const uint4*>(vc + ((static_cast<int64_t>(bt[key / bs]) * G + g) * bs + key % bs) * V + cc);
              }
            }
          }
#pragma unroll
          for (int p = 0; p < 4; ++p) {
            const int u = u0 + p * kThreads + tid;
            if (u < BK * kper) {
              const int j = u / kper, c = (u - j * kper) * 8;
              *reinterpret_cast<uint4*>(ks + j * DSH + c) = v[p];
            } else if (u < units) {
              const int u2 = u - BK * kper;
              const int j = u2 / vper, c = (u2 - j * vper) * 8;
              *reinterpret_cast<uint4*>(vs + j * VSH + c) = v[p];
            }
          }
        }
      }
      __syncthreads();
      for (int kb = w; kb < BK / 16; kb += kThreads / 64) {
        pk::f32x4 c4 = pk::f32x4{0.f, 0.f, 0.f, 0.f};
        const bf16_t* qr = qs + n * DSH + 8 * g4;
        const bf16_t* kr = ks + (kb * 16 + n) * DSH + 8 * g4;
        for (int kk = 0; kk < D / 32; ++kk)
          c4 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pk::ld8(qr + kk * 32), pk::ld8(kr + kk * 32), c4, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 4; ++i) ps[(4 * g4 + i) * BK + kb * 16 + n] = c4[i];
      }
      __syncthreads();
      float tmax = -INFINITY;
      for (int j = kg; j < BK; j += 16) {
        const int key = k0 + j;
        const bool seen = j < nk && live && (part == 0 ? key < my_blocks : (key <= my_pos && key >= my_lo));
        float d = -INFINITY;
        if (seen) {
          d = ps[qi * BK + j] * a.scale;
          if (a.softcap > 0.f) d = a.softcap * tanhf(d / a.softcap);
        }
        ps[qi * BK + j] = d;
        tmax = fmaxf(tmax, d);
      }
#pragma unroll
      for (int o = 8; o > 0; o >>= 1) tmax = fmaxf(tmax, __shfl_xor(tmax, o, 64));
      const float m_old = m_s[qi];
      const float m_new = fmaxf(m_old, tmax);
      float tsum = 0.f;
      for (int j = kg; j < BK; j += 16) {
        const float sc = ps[qi * BK + j];
        const float p = (m_new == -INFINITY || sc == -INFINITY) ? 0.f : expf(sc - m_new);
        const bf16_t hi = pk::f2bf(p);  // p = hi + lo to 16 bits: the weights meet the values at fp32-like precision
        pb[qi * PSH + j] = hi;
        pb2[qi * PSH + j] = pk::f2bf(p - pk::bf2f(hi));
        tsum += p;
      }
#pragma unroll
      for (int o = 8; o > 0; o >>= 1) tsum += __shfl_xor(tsum, o, 64);
      const float resc = (m_old == -INFINITY) ? 0.f : expf(m_old - m_new);
      if (kg == 0) r_s[qi] = resc;
      __syncthreads();
      if (kg == 0) {
        m_s[qi] = m_new;
        l_s[qi] = l_s[qi] * resc + tsum;
      }
      {
        float rs[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) rs[e] = r_s[4 * g4 + e];
#pragma unroll
        for (int i = 0; i < NV; ++i)
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[i][e] *= rs[e];
        for (int k32 = 0; k32 < BK / 32; ++k32) {
          const pk::bf16x8_t pa = pk::ld8(pb + n * PSH + k32 * 32 + 8 * g4);
          const pk::bf16x8_t pa2 = pk::ld8(pb2 + n * PSH + k32 * 32 + 8 * g4);
#pragma unroll
          for (int i = 0; i < NV; ++i) {
            const int col = (w + 4 * i) * 16 + n;
            if ((w + 4 * i) * 16 < VW) {
              const bf16_t* vr = vs + (k32 * 32 + 8 * g4) * VSH + col;
              pk::u32x4 bw;
#pragma unroll
              for (int e = 0; e < 4; ++e)
                bw[e] = static_cast<uint32_t>(vr[(2 * e) * VSH]) | (static_cast<uint32_t>(vr[(2 * e + 1) * VSH]) << 16);
              const pk::bf16x8_t vb = __builtin_bit_cast(pk::bf16x8_t, bw);
              acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa, vb, acc[i], 0, 0, 0);
              acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa2, vb, acc[i], 0, 0, 0);
            }
          }
        }
      }
      __syncthreads();
    }
  }
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int row = row0 + 4 * g4 + e;
    if (row >= n_rows) break;
    const int tl = row / R, h = kh * R + row - tl * R;
    const float l = l_s[4 * g4 + e];
    if (a.n_parts > 1) {
      const int64_t slot = (static_cast<int64_t>(q0 + tl) * H + h) * a.n_parts + blockIdx.z;
      float* dst = a.ws_acc + slot * VW;
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int c = (w + 4 * i) * 16 + n;
        if (c < VW) dst[c] = acc[i][e];
      }
      if (w == 0 && n == 0) {
        a.ws_ml[2 * slot] = m_s[4 * g4 + e];
        a.ws_ml[2 * slot + 1] = l;
      }
    } else {
      const float inv = l > 0.f ? 1.f / l : 0.f;
      float* dst = a.out + (static_cast<int64_t>(q0 + tl) * H + h) * VW;
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int c = (w + 4 * i) * 16 + n;
        if (c < VW) dst[c] = acc[i][e] * inv;
      }
    }
  }
}

size_t mfma_lds_bytes(int D, int VW, int bk) {
  return (static_cast<size_t>(kBQ) * (D + 8) + static_cast<size_t>(bk) * (D + 8 + VW + 8) + 2 * kBQ * (bk + 8)) * 2 +
         (static_cast<size_t>(kBQ) * bk + 3 * kBQ) * 4;
}

int g_pooled_mfma = 1;  // 0: every launch takes the FMA kernel (tests compare the two)

// out[t, h] from the parts' (max, sum, unnormalised sums) and the head's sink: one wave per (token, head)
__global__ void __launch_bounds__(64)
pooled_merge_kernel(float* __restrict__ out, const float* __restrict__ ws_acc, const float* __restrict__ ws_ml,
                    const float* __restrict__ sink, int H, int VW, int n_parts) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int64_t row = static_cast<int64_t>(t) * H + h;
  const float* ml = ws_ml + row * n_parts * 2;
  float m = sink ? sink[h] : -INFINITY;
  for (int p = 0; p < n_parts; ++p) m = fmaxf(m, ml[2 * p]);
  float l = (sink && m != -INFINITY) ? expf(sink[h] - m) : 0.f;
  for (int p = 0; p < n_parts; ++p)
    if (ml[2 * p] != -INFINITY) l += ml[2 * p + 1] * expf(ml[2 * p] - m);
  const float inv = l > 0.f ? 1.f / l : 0.f;
  for (int c = lane; c < VW; c += 64) {
    float acc = 0.f;
    for (int p = 0; p < n_parts; ++p)
      if (ml[2 * p] != -INFINITY) acc += ws_acc[(row * n_parts + p) * VW + c] * expf(ml[2 * p] - m);
    out[row * VW + c] = acc * inv;
  }
}

size_t lds_bytes(int D, int VW, int bk) {
  return (static_cast<size_t>(kBQ) * (D + 1) + static_cast<size_t>(bk) * (D + 1 + VW + 1) + kBQ * bk + 3 * kBQ) * 4;
}

// key tile: the largest of 64 / 32 / 16 whose tiles fit 60 KiB of LDS, else the largest of 32 / 16 / 8
// within 144 KiB; 0: the heads are too wide
int key_tile(int D, int VW) {
  for (int bk = 64; bk >= 16; bk >>= 1)
    if (lds_bytes(D, VW, bk) <= 60 * 1024) return bk;
  for (int bk = 32; bk >= 8; bk >>= 1)
    if (lds_bytes(D, VW, bk) <= 144 * 1024) return bk;
  return 0;
}

template <typename T, int NV>
int launch_one(const PooledArgs& a, dim3 grid, size_t lds, hipStream_t stream) {
  if (lds > 60 * 1024) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(pooled_attention_kernel<T, NV>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
    if (e != hipSuccess) return static_cast<int>(e);
  }
  pooled_attention_kernel<T, NV><<<grid, kThreads, lds, stream>>>(a);
  return PK_CHECK_LAUNCH();
}

template <typename T>
int launch_pooled(const PooledArgs& a, dim3 grid, int VW, hipStream_t stream) {
  const size_t lds = lds_bytes(a.D, VW, a.BK);
  const int nv = (VW + 63) / 64;
  if (nv <= 1) return launch_one<T, 1>(a, grid, lds, stream);
  if (nv <= 2) return launch_one<T, 2>(a, grid, lds, stream);
  if (nv <= 4) return launch_one<T, 4>(a, grid, lds, stream);
  if (nv <= 8) return launch_one<T, 8>(a, grid, lds, stream);
  return launch_one<T, 16>(a, grid, lds, stream);
}

// one wave per (token, head)
template <typename OT>
__global__ void __launch_bounds__(64)
mix_heads_kernel(OT* __restrict__ out, int64_t out_stride, const float* __restrict__ o, const float* __restrict__ talk, int H,
                 int VG, int V, float post) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  OT* dst = out + static_cast<int64_t>(t) * out_stride + static_cast<int64_t>(h) * V;
  const float* row = o + static_cast<int64_t>(t) * H * VG * V;
  if (!talk) {
    for (int c = lane; c < V; c += 64) st<OT>(dst + c, post * row[static_cast<int64_t>(h) * VG * V + c]);
    return;
  }
  const int vh = h / (H / VG);
  for (int c = lane; c < V; c += 64) {
    float acc = 0.f;
    for (int g = 0; g < H; ++g) acc += talk[h * H + g] * row[(static_cast<int64_t>(g) * VG + vh) * V + c];
    st<OT>(dst + c, post * acc);
  }
}

}  // namespace

// caches [blocks, G, bs, D | V] of element type dt; a token at the last position of a block writes the block's means
// (not a token whose slot_mapping entry is negative: it caches nothing)
PK_EXPORT int pkm_pool_update(const void* k_cache, const void* v_cache, void* kp_cache, void* vp_cache,
                              const void* positions, const void* slot_mapping, const void* token_seq,
                              const void* block_tables, long long bt_stride,
                              int T, int G, int D, int V, int bs, int pool, int dt, hipStream_t stream) {
  if (T <= 0 || pool <= 0) return 0;
  if (G < 1 || D < 1 || V < 1 || bs < 1) return -1;
  const dim3 grid(T, G);
  PKM_DISPATCH(dt, E, pool_update_kernel<E><<<grid, 256, 0, stream>>>(
                          static_cast<const E*>(k_cache), static_cast<const E*>(v_cache), static_cast<E*>(kp_cache),
                          static_cast<E*>(vp_cache), static_cast<const int*>(positions),
                          static_cast<const int*>(slot_mapping), static_cast<const int*>(token_seq),
                          static_cast<const int*>(block_tables), bt_stride, G, D, V, bs, pool));
  return PK_CHECK_LAUNCH();
}

// out fp32 [T, H, VG, V] (VG = G with all_values, else 1); q [T, H, D]; kp / vp null with pool = 0; n_parts > 1:
// workspaces ws_acc [T * H, n_parts, VG * V] and ws_ml [T * H, n_parts, 2] fp32
PK_EXPORT int pkm_pooled_attention(void* out, const void* q, const void* k_cache, const void* v_cache, const void* kp_cache,
                                   const void* vp_cache, const void* block_tables, long long bt_stride, const void* cu_q,
                                   const void* context_lens, const void* sink, int n_seqs, int T, int H, int G, int D, int V,
                                   int bs, float scale, float softcap, int window, int pool, int all_values, int n_parts,
                                   void* ws_acc, void* ws_ml, int dt, hipStream_t stream) {
  if (T <= 0 || n_seqs <= 0) return 0;
  if (H < 1 || G < 1 || H % G || D < 1 || V < 1 || bs < 1 || window < 0 || pool < 0) return -1;
  if (pool > 0 && (!kp_cache || !vp_cache || window <= 0)) return -1;
  const int VW = (all_values ? G : 1) * V;
  if (VW > 1024) return -1;
  PooledArgs a{static_cast<float*>(out), q, k_cache, v_cache, kp_cache, vp_cache, static_cast<const int*>(block_tables),
               bt_stride, static_cast<const int*>(cu_q), static_cast<const int*>(context_lens),
               static_cast<const float*>(sink), n_seqs, H, G, D, V, bs, key_tile(D, VW), scale, softcap, window, pool,
               all_values, n_parts, static_cast<float*>(ws_acc), static_cast<float*>(ws_ml)};
  if (a.BK == 0 || n_parts < 1 || n_parts > 64 || (n_parts > 1 && (!ws_acc || !ws_ml))) return -1;
  const int R = H / G;
  // an upper bound of the row tiles: every sequence's rows rounded up
  const int tiles = (T * R + kBQ - 1) / kBQ + n_seqs;
  const dim3 grid(tiles, G, n_parts);
  int rc = -2;
  // bf16 with sizes the matrix-core tiles take: 32-key tiles within the default LDS limit
  if (dt == kBF16 && g_pooled_mfma && D % 32 == 0 && V % 8 == 0 && VW % 16 == 0 && mfma_lds_bytes(D, VW, 32) <= 144 * 1024) {
    a.BK = 32;
    const size_t lds = mfma_lds_bytes(D, VW, 32);
    const int nv = (VW + 63) / 64;
#define PKM_PM(NV)                                                                                                       \
  {                                                                                                                      \
    if (lds > 60 * 1024) {                                                                                               \
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(pooled_attention_mfma_kernel<NV>),          \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));        \
      if (e != hipSuccess) return static_cast<int>(e);                                                                   \
    }                                                                                                                    \
    pooled_attention_mfma_kernel<NV><<<grid, kThreads, lds, stream>>>(a);                                                \
  }
    if (nv <= 1) {
      PKM_PM(1);
    } else if (nv <= 2) {
      PKM_PM(2);
    } else if (nv <= 4) {
      PKM_PM(4);
    } else if (nv <= 8) {
      PKM_PM(8);
    } else {
      PKM_PM(16);
    }
#undef PKM_PM
    rc = PK_CHECK_LAUNCH();
  } else if (dt == kBF16) rc = launch_pooled<bf16_t>(a, grid, VW, stream);
  if (dt == kF32) rc = launch_pooled<float>(a, grid, VW, stream);
  if (rc != 0 || n_parts == 1) return rc;
  pooled_merge_kernel<<<dim3(T, H), 64, 0, stream>>>(a.out, a.ws_acc, a.ws_ml, a.sink, H, VW, n_parts);
  return PK_CHECK_LAUNCH();
}

PK_EXPORT int pkm_set_pooled_mfma(int on) {
  g_pooled_mfma = on;
  return 0;
}

// o fp32 [T, H, VG, V]; talk [H, H] fp32 (VG = G) or null (VG = 1); out rows out_stride elements apart
PK_EXPORT int pkm_mix_heads(void* out, long long out_stride, int out_dt, const void* o, const void* talk, int T, int H,
                            int VG, int V, float post, hipStream_t stream) {
  if (T <= 0) return 0;
  if (H < 1 || VG < 1 || H % VG || V < 1 || (talk == nullptr && VG != 1)) return -1;
  const dim3 grid(T, H);
  PKM_DISPATCH(out_dt, O, mix_heads_kernel<O><<<grid, 64, 0, stream>>>(static_cast<O*>(out), out_stride,
                                                                       static_cast<const float*>(o),
                                                                       static_cast<const float*>(talk), H, VG, V, post));
  return PK_CHECK_LAUNCH();
}

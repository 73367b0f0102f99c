// Softmax attention over a paged cache with a band of visible keys per query, learned sinks and
// separate counts of query, key and value heads; the rotations and cache writes in front of it; and
// the per-head norm / gate behind it.
//
//   rotate_cache      q and k heads turn by the token's position (fp32 (cos, sin) table rows; pair i
//                     = (i, i + pairs) or (2i, 2i + 1)); q -> [T, QH, D], k -> cache
//                     [blocks, KH, block_size, D], v -> cache [blocks, VH, block_size, V]
//   latent_in         a projection row [query latent | key / value latent | shared key part]: both
//                     latents set to unit RMS times a weight, the key part turned by the position;
//                     the query latent is returned, [latent | key part] goes to the cache row
//   latent_query      [folded query | the head's rotated part turned by the position]
//   masked_attention  query at position p sees keys lo(p) <= j <= p, lo(p) = max(0, p - window + 1,
//                     floor(p / chunk) chunk); p_j = exp(s_j) / (exp(sink_h) + sum_j' exp(s_j')),
//                     s = q . k * scale; o = sum_j p_j v_j.  Query head h reads key head h / (QH / KH)
//                     and value head h / (QH / VH); the value may be the first V numbers of the key row.
//   head_norm_gate    per (token, head): u / sqrt(mean(u^2) + eps) * w * post * act(gate), with u one
//                     head's row or the difference first - coef * second of two attention maps
//
// Scores, softmax, sums and norms are fp32 for both element types.  The (token, head) pairs of a
// sequence that share a key head are the rows of one tile problem against key / value tiles staged
// once in LDS; key tiles start at multiples of the tile size counted from key 0 of the sequence, so
// a position's sums run in the same order however its prompt was cut and whatever else the step holds.
#include "mix_common.h"

using namespace pkm;

namespace {

__device__ __forceinline__ int clamp_pos(int pos, int rows) { return pos < 0 ? 0 : (pos >= rows ? max(rows - 1, 0) : pos); }

// one wave turns one head: x[i], x[i + pairs] (halves) or x[2i], x[2i + 1] of the first 2 * pairs
// coordinates by (cos, sin) = cs[2i], cs[2i + 1]; the rest pass.  IN -> OUT element types.
// nw [D] fp32 or null: the head is first set to unit RMS (eps inside the root) times that weight.
template <typename IN, typename OUT>
__device__ __forceinline__ void turn_head(OUT* dst, const IN* src, int D, const float* cs, int pairs, int halves, int lane,
                                          const float* nw = nullptr, float eps = 0.f) {
  float k = 1.f;
  if (nw) {
    float ss = 0.f;
    for (int i = lane; i < D; i += 64) {
      const float x = ld<IN>(src + i);
      ss += x * x;
    }
    ss = pk::wave_sum(ss);
    k = 1.f / sqrtf(ss / static_cast<float>(D) + eps);
  }
  for (int i = lane; i < pairs; i += 64) {
    const int iu = halves ? i : 2 * i, iv = halves ? i + pairs : 2 * i + 1;
    float u = ld<IN>(src + iu), v = ld<IN>(src + iv);
    if (nw) {
      u = u * k * nw[iu];
      v = v * k * nw[iv];
    }
    const float c = cs[2 * i], s = cs[2 * i + 1];
    st<OUT>(dst + iu, u * c - v * s);
    st<OUT>(dst + iv, v * c + u * s);
  }
  for (int i = 2 * pairs + lane; i < D; i += 64) {
    const float x = ld<IN>(src + i);
    st<OUT>(dst + i, nw ? x * k * nw[i] : x);
  }
}

template <typename T>
__global__ void __launch_bounds__(64)
rotate_cache_kernel(T* __restrict__ q_out, const T* __restrict__ proj, int64_t stride, const int* __restrict__ positions,
                    const int* __restrict__ slot_mapping, const float* __restrict__ table, int pairs, int table_rows,
                    int halves, T* __restrict__ k_cache, T* __restrict__ v_cache, int QH, int KH, int VH, int D, int V,
                    int bs, const float* __restrict__ q_norm, const float* __restrict__ k_norm, float eps) {
  const int t = blockIdx.x, item = blockIdx.y, lane = threadIdx.x;
  const int slot = slot_mapping[t];
  const T* row = proj + static_cast<int64_t>(t) * stride;
  const float* cs = table ? table + static_cast<int64_t>(clamp_pos(positions[t], table_rows)) * pairs * 2 : nullptr;
  const int np = cs ? pairs : 0;
  if (item < QH) {
    turn_head<T, T>(q_out + (static_cast<int64_t>(t) * QH + item) * D, row + static_cast<int64_t>(item) * D, D, cs, np,
                    halves, lane, q_norm, eps);
  } else if (item < QH + KH) {
    if (slot < 0) return;
    const int g = item - QH;
    turn_head<T, T>(k_cache + ((static_cast<int64_t>(slot / bs) * KH + g) * bs + slot % bs) * D,
                    row + static_cast<int64_t>(item) * D, D, cs, np, halves, lane, k_norm, eps);
  } else {
    if (slot < 0) return;
    const int g = item - QH - KH;
    const T* src = row + static_cast<int64_t>(QH + KH) * D + static_cast<int64_t>(g) * V;
    T* dst = v_cache + ((static_cast<int64_t>(slot / bs) * VH + g) * bs + slot % bs) * V;
    for (int i = lane; i < V; i += 64) dst[i] = src[i];
  }
}

// blockIdx.y: 0 the query latent, 1 the key / value latent and the shared key part
template <typename T>
__global__ void __launch_bounds__(256)
latent_in_kernel(T* __restrict__ cq, T* __restrict__ cache, const T* __restrict__ proj, int64_t stride, int Q, int R, int Dr,
                 const float* __restrict__ wq, const float* __restrict__ wkv, float eps, const int* __restrict__ positions,
                 const int* __restrict__ slot_mapping, const float* __restrict__ table, int pairs, int table_rows,
                 int halves, int bs) {
  __shared__ float red[16];
  const int t = blockIdx.x, tid = threadIdx.x;
  const T* row = proj + static_cast<int64_t>(t) * stride;
  const bool query = blockIdx.y == 0;
  if (query && Q == 0) return;
  const int slot = slot_mapping[t];
  if (!query && slot < 0) return;
  const T* src = query ? row : row + Q;
  const int n = query ? Q : R;
  const float* w = query ? wq : wkv;
  T* dst = query ? cq + static_cast<int64_t>(t) * Q : cache + static_cast<int64_t>(slot) * (R + Dr);
  float ss = 0.f;
  for (int i = tid; i < n; i += 256) {
    const float v = ld<T>(src + i);
    ss += v * v;
  }
  ss = pk::block_sum(ss, red);
  const float k = 1.f / sqrtf(ss / static_cast<float>(n) + eps);
  for (int i = tid; i < n; i += 256) st<T>(dst + i, ld<T>(src + i) * k * w[i]);
  if (!query && tid < 64 && Dr > 0) {
    const float* cs = table ? table + static_cast<int64_t>(clamp_pos(positions[t], table_rows)) * pairs * 2 : nullptr;
    turn_head<T, T>(dst + R, src + R, Dr, cs, cs ? pairs : 0, halves, tid);
  }
}

template <typename T>
__global__ void __launch_bounds__(64)
latent_query_kernel(T* __restrict__ out, const T* __restrict__ q_lat, const T* __restrict__ q,
                    const int* __restrict__ positions, const float* __restrict__ table, int pairs, int table_rows,
                    int halves, int T_, int H, int R, int D, int Dr) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  T* dst = out + (static_cast<int64_t>(t) * H + h) * (R + Dr);
  const T* src = q_lat + (static_cast<int64_t>(h) * T_ + t) * R;
  for (int i = lane; i < R; i += 64) dst[i] = src[i];
  if (Dr > 0) {
    const float* cs = table ? table + static_cast<int64_t>(clamp_pos(positions[t], table_rows)) * pairs * 2 : nullptr;
    turn_head<T, T>(dst + R, q + (static_cast<int64_t>(t) * H + h) * (D + Dr) + D, Dr, cs, cs ? pairs : 0, halves, lane);
  }
}

constexpr int kBQ = 16;        // (token, head) rows per workgroup
constexpr int kThreads = 256;  // 16 rows x 16 lanes

struct MaskedArgs {
  void* out;
  int64_t out_ts, out_hs;  // element strides of a token and of a head in out
  int out_f32;
  const void* q;  // [T, QH, D]
  int q_f32;
  const void* k_cache;  // [blocks, KH, bs, D]
  const void* v_cache;  // [blocks, VH, bs, v_width]
  int v_width;
  const int* block_tables;
  int64_t bt_stride;
  const int* cu_q;
  const int* context_lens;
  const float* sink;  // [QH] logits or null
  int n_seqs, QH, KH, VH, D, V, bs, BK;
  float scale;
  int window, chunk;
  // decoded tokens on the matrix cores: the band's keys cut into n_parts runs of `part` keys,
  // partial sums in the workspace (merged by masked_merge_kernel)
  int part, n_parts;
  float* ws_o;   // [n_seqs, n_parts, QH, V] unnormalised
  float* ws_ml;  // [n_seqs, n_parts, QH, 2] (max in log2 units, sum)
};

__device__ __forceinline__ int first_key(int pos, int window, int chunk) {
  int lo = 0;
  if (window > 0) lo = max(lo, pos - window + 1);
  if (chunk > 0) lo = max(lo, pos / chunk * chunk);
  return lo;
}

// NV: output accumulators per thread = ceil(V / 16).  ALIAS: the value of a key is the first V
// numbers of its key row (KH == VH, same cache).
template <typename T, int NV, bool ALIAS>
__global__ void __launch_bounds__(kThreads) masked_attention_kernel(MaskedArgs a) {
  extern __shared__ float smem[];
  const int QH = a.QH, KH = a.KH, D = a.D, V = a.V, BK = a.BK, bs = a.bs;
  const int R = QH / KH;  // query heads per key head
  const int kh = blockIdx.y;
  const int vh = kh / (KH / a.VH);
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
  const int DS = D + 1, VS = V + 1;  // odd row strides: conflict-free column walks
  float* qs = smem;                  // [kBQ][DS]
  float* ks = qs + kBQ * DS;         // [BK][DS]
  float* vs = ALIAS ? ks : ks + BK * DS;           // [BK][VS] (ALIAS: the key rows)
  float* ps = ALIAS ? ks + BK * DS : vs + BK * VS;  // [kBQ][BK]
  float* m_s = ps + kBQ * BK;        // [kBQ] running max
  float* l_s = m_s + kBQ;            // [kBQ] running sum
  const int vstride = ALIAS ? DS : VS;
  const int tid = threadIdx.x;
  const int qi = tid >> 4, kg = tid & 15;
  const int* bt = a.block_tables + static_cast<int64_t>(s) * a.bt_stride;
  const T* kc = static_cast<const T*>(a.k_cache);
  const T* vc = static_cast<const T*>(a.v_cache);

  for (int e = tid; e < kBQ * D; e += kThreads) {
    const int r = e / D, c = e - r * D;
    const int row = row0 + r;
    float v = 0.f;
    if (row < n_rows) {
      const int tl = row / R, h = kh * R + row - tl * R;
      const int64_t at = (static_cast<int64_t>(q0 + tl) * QH + h) * D + c;
      v = a.q_f32 ? static_cast<const float*>(a.q)[at] : ld<T>(static_cast<const T*>(a.q) + at);
    }
    qs[r * DS + c] = v;
  }
  const int my_row = row0 + qi;
  const bool live = my_row < n_rows;
  const int my_tl = live ? my_row / R : 0;
  const int my_h = kh * R + (live ? my_row - my_tl * R : 0);
  const int my_pos = live ? ctx - qlen + my_tl : -1;
  const int my_lo = live ? first_key(my_pos, a.window, a.chunk) : 0;
  if (tid < kBQ) {
    const int row = row0 + tid;
    const int h = kh * R + (row < n_rows ? row % R : 0);
    m_s[tid] = a.sink ? a.sink[h] : -INFINITY;  // the sink is a key without a value
    l_s[tid] = a.sink ? 1.f : 0.f;
  }
  const int first_pos = ctx - qlen + row0 / R;
  const int last_pos = ctx - qlen + (min(row0 + kBQ, n_rows) - 1) / R;
  const int k_end = last_pos + 1;  // keys [k_begin, k_end) are visible to some row
  const int k_begin = first_pos >= 0 ? first_key(first_pos, a.window, a.chunk) / BK * BK : 0;
  float acc[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) acc[i] = 0.f;
  __syncthreads();

  for (int k0 = k_begin; k0 < k_end; k0 += BK) {
    const int nk = min(BK, k_end - k0);
    for (int e = tid; e < BK * D; e += kThreads) {
      const int j = e / D, c = e - j * D;
      float v = 0.f;
      if (j < nk) {
        const int key = k0 + j;
        v = ld<T>(kc + ((static_cast<int64_t>(bt[key / bs]) * KH + kh) * bs + key % bs) * D + c);
      }
      ks[j * DS + c] = v;
    }
    if (!ALIAS) {
      for (int e = tid; e < BK * V; e += kThreads) {
        const int j = e / V, c = e - j * V;
        float v = 0.f;
        if (j < nk) {
          const int key = k0 + j;
          v = ld<T>(vc + ((static_cast<int64_t>(bt[key / bs]) * a.VH + vh) * bs + key % bs) * a.v_width + c);
        }
        vs[j * VS + c] = v;
      }
    }
    __syncthreads();
    float tmax = -INFINITY;
    for (int j = kg; j < BK; j += 16) {
      float d = 0.f;
      const float* qr = qs + qi * DS;
      const float* kr = ks + j * DS;
      for (int c = 0; c < D; ++c) d += qr[c] * kr[c];
      d *= a.scale;
      const int key = k0 + j;
      d = (j < nk && key <= my_pos && key >= my_lo) ? d : -INFINITY;
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
    __syncthreads();  // every lane of the row has read m_old and its own scores
    if (kg == 0) {
      m_s[qi] = m_new;
      l_s[qi] = l_s[qi] * resc + tsum;
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) acc[i] *= resc;
    for (int j = 0; j < nk; ++j) {
      const float p = ps[qi * BK + j];
      const float* vr = vs + j * vstride + kg;
#pragma unroll
      for (int i = 0; i < NV; ++i)
        if (kg + 16 * i < V) acc[i] += p * vr[16 * i];
    }
    __syncthreads();
  }
  const float l = l_s[qi];
  const float inv = l > 0.f ? 1.f / l : 0.f;
  if (!live) return;
  const int64_t at = static_cast<int64_t>(q0 + my_tl) * a.out_ts + static_cast<int64_t>(my_h) * a.out_hs;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = kg + 16 * i;
    if (c < V) {
      if (a.out_f32) {
        static_cast<float*>(a.out)[at + c] = acc[i] * inv;
      } else {
        st<T>(static_cast<T*>(a.out) + at + c, acc[i] * inv);
      }
    }
  }
}

size_t lds_bytes(int D, int V, int bk, bool alias) {
  return (static_cast<size_t>(kBQ) * (D + 1) + static_cast<size_t>(bk) * (D + 1 + (alias ? 0 : V + 1)) + kBQ * bk + 2 * kBQ) * 4;
}

// key tile: the largest of 64 / 32 / 16 whose tiles fit 60 KiB of LDS, else the largest of 32 / 16 / 8
// within 144 KiB; 0: the heads are too wide
int key_tile(int D, int V, bool alias) {
  for (int bk = 64; bk >= 16; bk >>= 1)
    if (lds_bytes(D, V, bk, alias) <= 60 * 1024) return bk;
  for (int bk = 32; bk >= 8; bk >>= 1)
    if (lds_bytes(D, V, bk, alias) <= 144 * 1024) return bk;
  return 0;
}

template <typename T, int NV, bool ALIAS>
int launch_one(const MaskedArgs& a, dim3 grid, size_t lds, hipStream_t stream) {
  if (lds > 60 * 1024) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(masked_attention_kernel<T, NV, ALIAS>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
    if (e != hipSuccess) return static_cast<int>(e);
  }
  masked_attention_kernel<T, NV, ALIAS><<<grid, kThreads, lds, stream>>>(a);
  return PK_CHECK_LAUNCH();
}

template <typename T, bool ALIAS>
int launch_masked(const MaskedArgs& a, dim3 grid, hipStream_t stream) {
  const size_t lds = lds_bytes(a.D, a.V, a.BK, ALIAS);
  const int nv = (a.V + 15) / 16;
  if (nv <= 1) return launch_one<T, 1, ALIAS>(a, grid, lds, stream);
  if (nv <= 2) return launch_one<T, 2, ALIAS>(a, grid, lds, stream);
  if (nv <= 4) return launch_one<T, 4, ALIAS>(a, grid, lds, stream);
  if (nv <= 8) return launch_one<T, 8, ALIAS>(a, grid, lds, stream);
  if (nv <= 16) return launch_one<T, 16, ALIAS>(a, grid, lds, stream);
  return launch_one<T, 32, ALIAS>(a, grid, lds, stream);
}

// ---- bf16 on the matrix cores -------------------------------------------------------------------
// NW waves of 16 (token, head) rows of one key head against 32-key tiles staged in LDS (pages hold
// whole 32-key tiles; a tile is one contiguous run of the key cache).  Both products run transposed
// on mfma_f32_16x16x32_bf16 so that the softmax weights never leave their registers:
//
//   S^T [keys x rows] = K [keys x D] . Q^T      A = key rows from LDS, B = the wave's Q (registers)
//   O^T [V x rows]   += V^T [V x keys] . P^T    A = value columns from LDS, B = P^T from the S^T accumulators
//
// An accumulator lane (g4, n) holds query row n and keys 4 g4 .. 4 g4 + 3 of each 16-key half; the B
// operand of the second product wants 8 key slots per lane, so slot (g4, e) is key 4 g4 + e of the
// first half for e < 4 and key 16 + 4 g4 + e - 4 of the second.  The caches are key-major, so a
// thread turns 4 keys x 8 value columns in registers and writes 8 column words of 4 keys into the
// column-major LDS tile at those slots.  Scores are kept in log2 units.  Tiles of the next step are
// fetched into registers before the current products.  A wave skips tiles outside its rows' bands.
// Row tiles are dealt to the XCDs in contiguous ranges, so tiles that share keys share an L2.
constexpr float kLog2e = 1.4426950408889634f;

__host__ __device__ __forceinline__ int quad_slot(int q) { return (q & 3) * 8 + 4 * (q >> 2); }  // slot of key 4 q

// SPLIT: one token per sequence; blockIdx.z picks a run of a.part keys of the band and the
// workgroup leaves (max, sum, unnormalised o) per row in the workspace (no sink: the merge adds it).
template <int D, int V, int NW, bool ALIAS, bool SPLIT>
__global__ void __launch_bounds__(64 * NW) masked_attention_mfma_kernel(MaskedArgs a) {
  constexpr int NT = 64 * NW, BQ = 16 * NW, BK = 32, NKK = D / 32, NRT = V / 16, CS = D + 8, CT = BK + 8;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16_t* ks = reinterpret_cast<bf16_t*>(smem_raw);  // [BK][CS]  key-major
  bf16_t* vt = ks + BK * CS;                          // [V][CT]   column-major, key slots permuted
  const int QH = a.QH, KH = a.KH, bs = a.bs, R = QH / KH;
  const int kh = blockIdx.y, vh = kh / (KH / a.VH);
  int s = 0, tile = blockIdx.x;
  if (SPLIT) {
    const int ntile = (R + BQ - 1) / BQ;
    s = blockIdx.x / ntile;
    tile = blockIdx.x - s * ntile;
  } else {
    // workgroups go to the 8 XCDs round-robin: XCD x takes the x-th eighth of the row tiles (gridDim.x
    // is a multiple of 8), so neighbouring tiles, which share most of their keys, share one L2
    tile = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
    for (; s < a.n_seqs; ++s) {
      const int nt = ((a.cu_q[s + 1] - a.cu_q[s]) * R + BQ - 1) / BQ;
      if (tile < nt) break;
      tile -= nt;
    }
    if (s >= a.n_seqs) return;
  }
  const int q0 = a.cu_q[s], qlen = a.cu_q[s + 1] - q0, ctx = a.context_lens[s];
  const int n_rows = qlen * R, row0 = tile * BQ;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = lane >> 4, n = lane & 15;
  const int* bt = a.block_tables + static_cast<int64_t>(s) * a.bt_stride;
  const int my_row = row0 + 16 * wave + n;
  const bool valid = my_row < n_rows;
  const int tl = valid ? my_row / R : 0, h = kh * R + (valid ? my_row - tl * R : 0);
  const int my_pos = valid ? ctx - qlen + tl : -1;
  const int my_lo = valid ? first_key(my_pos, a.window, a.chunk) : 0x7fffffff;
  const int first_pos = ctx - qlen + row0 / R;
  int max_pos = ctx - qlen + (min(row0 + BQ, n_rows) - 1) / R;
  int k_begin = first_pos >= 0 ? first_key(first_pos, a.window, a.chunk) / BK * BK : 0;
  if (SPLIT) {
    k_begin += blockIdx.z * a.part;
    max_pos = min(max_pos, k_begin + a.part - 1);
  }
  const bf16_t* q = static_cast<const bf16_t*>(a.q);
  const bf16_t* kc = static_cast<const bf16_t*>(a.k_cache);
  const bf16_t* vc = static_cast<const bf16_t*>(a.v_cache);
  const float sl2 = a.scale * kLog2e;

  pk::bf16x8_t qf[NKK];
  {
    const bf16_t* qr = q + (static_cast<int64_t>(q0 + tl) * QH + h) * D + 8 * g;
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) {
      pk::u32x4 v = {0u, 0u, 0u, 0u};
      if (valid) v = *reinterpret_cast<const pk::u32x4*>(qr + kk * 32);
      qf[kk] = __builtin_bit_cast(pk::bf16x8_t, v);
    }
  }
  pk::f32x4 o[NRT];
#pragma unroll
  for (int rt = 0; rt < NRT; ++rt) o[rt] = pk::f32x4{0.f, 0.f, 0.f, 0.f};
  const bool with_sink = !SPLIT && a.sink != nullptr;
  float m_run = with_sink ? a.sink[h] * kLog2e : -INFINITY, l_run = with_sink ? 1.f : 0.f;

  constexpr int KCH = BK * D / 8;          // 16-byte chunks of a key tile
  constexpr int KIT = (KCH + NT - 1) / NT;
  constexpr int VUN = V;                   // units of (4 keys x 8 value columns): 8 quads x V / 8 column chunks
  constexpr int VIT = (VUN + NT - 1) / NT;
  pk::u32x4 kv[KIT], vv[VIT][4];
  auto fetch = [&](int k0) {
    const int64_t blk = bt[k0 / bs];
    const bf16_t* ksrc = kc + ((blk * KH + kh) * bs + k0 % bs) * D;
    const bf16_t* vsrc = vc + ((blk * a.VH + vh) * bs + k0 % bs) * a.v_width;
#pragma unroll
    for (int i = 0; i < KIT; ++i) {
      const int c = tid + NT * i;
      if (c < KCH) kv[i] = *reinterpret_cast<const pk::u32x4*>(ksrc + c * 8);
    }
#pragma unroll
    for (int i = 0; i < VIT; ++i) {
      const int u = tid + NT * i;
      if (u < VUN) {
        const int qd = u & 7, c8 = u >> 3;
#pragma unroll
        for (int j = 0; j < 4; ++j)
          vv[i][j] = *reinterpret_cast<const pk::u32x4*>(vsrc + static_cast<int64_t>(4 * qd + j) * a.v_width + c8 * 8);
      }
    }
  };
  if (k_begin <= max_pos) fetch(k_begin);
  for (int k0 = k_begin; k0 <= max_pos; k0 += BK) {
#pragma unroll
    for (int i = 0; i < KIT; ++i) {
      const int c = tid + NT * i;
      if (c < KCH) {
        const int key = c / (D / 8), d8 = c - key * (D / 8);
        *reinterpret_cast<pk::u32x4*>(ks + key * CS + d8 * 8) = kv[i];
      }
    }
#pragma unroll
    for (int i = 0; i < VIT; ++i) {
      const int u = tid + NT * i;
      if (u < VUN) {
        const int qd = u & 7, c8 = u >> 3;
        bf16_t* dst = vt + (c8 * 8) * CT + quad_slot(qd);
#pragma unroll
        for (int w = 0; w < 4; ++w) {  // columns 2 w (low halves) and 2 w + 1 (high halves) of the chunk
          uint2 lo, hi;
          lo.x = (vv[i][0][w] & 0xffffu) | (vv[i][1][w] << 16);
          lo.y = (vv[i][2][w] & 0xffffu) | (vv[i][3][w] << 16);
          hi.x = (vv[i][0][w] >> 16) | (vv[i][1][w] & 0xffff0000u);
          hi.y = (vv[i][2][w] >> 16) | (vv[i][3][w] & 0xffff0000u);
          *reinterpret_cast<uint2*>(dst + (2 * w) * CT) = lo;
          *reinterpret_cast<uint2*>(dst + (2 * w + 1) * CT) = hi;
        }
      }
    }
    __syncthreads();
    if (k0 + BK <= max_pos) fetch(k0 + BK);
    if (__any(my_pos >= k0 && my_lo <= k0 + BK - 1)) {
      pk::f32x4 sa[2] = {pk::f32x4{0.f, 0.f, 0.f, 0.f}, pk::f32x4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
      for (int sub = 0; sub < 2; ++sub) {
        const bf16_t* kr = ks + (sub * 16 + n) * CS + 8 * g;
#pragma unroll
        for (int kk = 0; kk < NKK; ++kk)
          sa[sub] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pk::ld8(kr + kk * 32), qf[kk], sa[sub], 0, 0, 0);
      }
      float sc[8];
      float tmax = -INFINITY;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int key = k0 + (e >> 2) * 16 + 4 * g + (e & 3);
        sc[e] = (key <= my_pos && key >= my_lo) ? sa[e >> 2][e & 3] * sl2 : -INFINITY;
        tmax = fmaxf(tmax, sc[e]);
      }
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
      const float m_new = fmaxf(m_run, tmax);
      float p[8], tsum = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        p[e] = sc[e] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(sc[e] - m_new);
        tsum += p[e];
      }
      tsum += __shfl_xor(tsum, 16, 64);
      tsum += __shfl_xor(tsum, 32, 64);
      const float resc = m_run == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m_run - m_new);
      m_run = m_new;
      l_run = l_run * resc + tsum;
      pk::u32x4 pw;
#pragma unroll
      for (int e = 0; e < 4; ++e) pw[e] = pk::pack2(p[2 * e], p[2 * e + 1]);
      const pk::bf16x8_t pb = __builtin_bit_cast(pk::bf16x8_t, pw);
      if (__any(resc != 1.f)) {
#pragma unroll
        for (int rt = 0; rt < NRT; ++rt) o[rt] *= resc;
      }
      const bf16_t* vr = vt + n * CT + 8 * g;
#pragma unroll
      for (int rt = 0; rt < NRT; ++rt)
        o[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pk::ld8(vr + rt * 16 * CT), pb, o[rt], 0, 0, 0);
    }
    __syncthreads();
  }
  if (SPLIT) {
    if (valid) {
      const int64_t at = (static_cast<int64_t>(s) * a.n_parts + blockIdx.z) * QH + h;
#pragma unroll
      for (int rt = 0; rt < NRT; ++rt)
        *reinterpret_cast<float4*>(a.ws_o + at * V + rt * 16 + 4 * g) = float4{o[rt][0], o[rt][1], o[rt][2], o[rt][3]};
      if (g == 0) {
        a.ws_ml[at * 2] = m_run;
        a.ws_ml[at * 2 + 1] = l_run;
      }
    }
    return;
  }
  if (valid) {
    const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
    const int64_t at = static_cast<int64_t>(q0 + tl) * a.out_ts + static_cast<int64_t>(h) * a.out_hs + 4 * g;
#pragma unroll
    for (int rt = 0; rt < NRT; ++rt) {
      const float w0 = o[rt][0] * inv, w1 = o[rt][1] * inv, w2 = o[rt][2] * inv, w3 = o[rt][3] * inv;
      if (a.out_f32) {
        *reinterpret_cast<float4*>(static_cast<float*>(a.out) + at + rt * 16) = float4{w0, w1, w2, w3};
      } else {
        uint2 w;
        w.x = pk::pack2(w0, w1);
        w.y = pk::pack2(w2, w3);
        *reinterpret_cast<uint2*>(static_cast<bf16_t*>(a.out) + at + rt * 16) = w;
      }
    }
  }
}

// out[token of sequence s, head h] from the runs' (max, sum, o) and the head's sink: one workgroup
// per (sequence, head); the first wave turns the (at most 64) runs into one weight per run.
template <typename T>
__global__ void __launch_bounds__(128)
masked_merge_kernel(void* __restrict__ out, int64_t out_ts, int64_t out_hs, int out_f32, const float* __restrict__ ws_o,
                    const float* __restrict__ ws_ml, const int* __restrict__ cu_q, const float* __restrict__ sink,
                    int n_parts, int QH, int V) {
  __shared__ float wgt[64];
  const int s = blockIdx.x, h = blockIdx.y;
  const int tok = cu_q[s];
  if (threadIdx.x < 64) {
    const int p = threadIdx.x;
    const int64_t at = (static_cast<int64_t>(s) * n_parts + p) * QH + h;
    const float m = p < n_parts ? ws_ml[at * 2] : -INFINITY;
    const float l = p < n_parts ? ws_ml[at * 2 + 1] : 0.f;
    const float sk = sink ? sink[h] * kLog2e : -INFINITY;
    const float M = pk::wave_max(fmaxf(m, sk));
    const float w = m == -INFINITY ? 0.f : exp2f(m - M);
    float L = pk::wave_sum(w * l);
    if (sink) L += exp2f(sk - M);
    wgt[p] = L > 0.f ? w / L : 0.f;
  }
  __syncthreads();
  const int64_t at = static_cast<int64_t>(tok) * out_ts + static_cast<int64_t>(h) * out_hs;
  const float* base = ws_o + (static_cast<int64_t>(s) * n_parts * QH + h) * V;
  for (int c = threadIdx.x; c < V; c += blockDim.x) {
    float u = 0.f;
    for (int p = 0; p < n_parts; ++p) u += wgt[p] * base[static_cast<int64_t>(p) * QH * V + c];
    if (out_f32) {
      static_cast<float*>(out)[at + c] = u;
    } else {
      st<T>(static_cast<T*>(out) + at + c, u);
    }
  }
}

template <int D, int V, int NW, bool ALIAS, bool SPLIT>
int launch_mfma_one(const MaskedArgs& a, int T, hipStream_t stream) {
  constexpr size_t lds = (32 * (D + 8) + V * 40) * sizeof(bf16_t);
  auto kern = masked_attention_mfma_kernel<D, V, NW, ALIAS, SPLIT>;
  if (lds > 60 * 1024) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                             static_cast<int>(lds));
    if (e != hipSuccess) return static_cast<int>(e);
  }
  const int R = a.QH / a.KH;
  const dim3 grid = SPLIT ? dim3(a.n_seqs * ((R + 16 * NW - 1) / (16 * NW)), a.KH, a.n_parts)
                          : dim3(((T * R + 16 * NW - 1) / (16 * NW) + a.n_seqs + 7) / 8 * 8, a.KH);
  kern<<<grid, 64 * NW, lds, stream>>>(a);
  return PK_CHECK_LAUNCH();
}

// head sizes the matrix-core kernel is built for
bool mfma_sizes(int D, int V, bool alias) {
  if (!alias) return (D == 64 || D == 128) && (V == 64 || V == 128);
  return (D == 96 && V == 64) || (D == 160 && V == 128) || (D == 192 && V == 128) || (D == 288 && V == 256) ||
         (D == 320 && V == 256) || (D == 576 && V == 512);
}

// returns -100 when the sizes are not among those the matrix-core kernel is built for
template <bool SPLIT>
int launch_mfma(const MaskedArgs& a, int T, bool alias, hipStream_t stream) {
#define PKM_MM(DD, VV, NW, NWS, AL) \
  if (a.D == DD && a.V == VV && alias == AL) return launch_mfma_one<DD, VV, (SPLIT ? NWS : NW), AL, SPLIT>(a, T, stream);
  // waves per workgroup for prompt portions / for decoded tokens (one 16-row tile computes there:
  // fewer, less loaded waves stage the tiles faster for the wide rows)
  PKM_MM(64, 64, 8, 8, false)
  PKM_MM(64, 128, 8, 8, false)
  PKM_MM(128, 64, 8, 8, false)
  PKM_MM(128, 128, 8, 8, false)
  PKM_MM(96, 64, 8, 8, true)
  PKM_MM(160, 128, 8, 8, true)
  PKM_MM(192, 128, 8, 8, true)
  PKM_MM(288, 256, 8, 4, true)
  PKM_MM(320, 256, 8, 4, true)
  PKM_MM(576, 512, 8, 4, true)
#undef PKM_MM
  return -100;
}

int g_masked_mfma = 1;  // 0: every launch takes the FMA kernel (tests compare the two)

constexpr int kGateNone = 0, kGateSigmoid = 1, kGateSilu = 2;

// one wave per (token, head)
template <typename GT, typename OT>
__global__ void __launch_bounds__(64)
head_norm_gate_kernel(OT* __restrict__ out, int64_t out_stride, const float* __restrict__ a, int H, int V, float eps,
                      const GT* __restrict__ gate, int64_t gate_stride, int gate_kind, const float* __restrict__ weight,
                      int weight_hs, float post, int pair_group, float coef) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const float *u1, *u2 = nullptr;
  if (pair_group > 0) {
    const int g = h / pair_group, j = h - g * pair_group;
    u1 = a + (static_cast<int64_t>(t) * 2 * H + static_cast<int64_t>(g) * 2 * pair_group + j) * V;
    u2 = u1 + static_cast<int64_t>(pair_group) * V;
  } else {
    u1 = a + (static_cast<int64_t>(t) * H + h) * V;
  }
  float ss = 0.f;
  for (int i = lane; i < V; i += 64) {
    const float u = u2 ? u1[i] - coef * u2[i] : u1[i];
    ss += u * u;
  }
  ss = pk::wave_sum(ss);
  const float k = post / sqrtf(ss / static_cast<float>(V) + eps);
  OT* dst = out + static_cast<int64_t>(t) * out_stride + static_cast<int64_t>(h) * V;
  if (weight) weight += static_cast<int64_t>(h) * weight_hs;
  const GT* gr = gate ? gate + static_cast<int64_t>(t) * gate_stride + static_cast<int64_t>(h) * V : nullptr;
  for (int i = lane; i < V; i += 64) {
    float z = (u2 ? u1[i] - coef * u2[i] : u1[i]) * k;
    if (weight) z *= weight[i];
    if (gr && gate_kind != kGateNone) {
      const float g = ld<GT>(gr + i);
      z *= gate_kind == kGateSigmoid ? sigmoidf(g) : g * sigmoidf(g);
    }
    st<OT>(dst + i, z);
  }
}

}  // namespace

// proj [T, QH*D | KH*D | VH*V] rows `stride` elements apart; table [table_rows, pairs, 2] fp32 or null;
// q_norm / k_norm [D] fp32 or null: unit RMS times the weight before the rotation
PK_EXPORT int pkm_rotate_cache(void* q_out, const void* proj, long long stride, const void* positions,
                               const void* slot_mapping, const void* table, int pairs, int table_rows, int halves,
                               void* k_cache, void* v_cache, int T, int QH, int KH, int VH, int D, int V, int bs,
                               const void* q_norm, const void* k_norm, float eps, int dt, hipStream_t stream) {
  if (T <= 0) return 0;
  if (D < 1 || V < 1 || 2 * pairs > D || (table && table_rows < 1) || bs < 1) return -1;
  const dim3 grid(T, QH + KH + VH);
  PKM_DISPATCH(dt, E, rotate_cache_kernel<E><<<grid, 64, 0, stream>>>(
                          static_cast<E*>(q_out), static_cast<const E*>(proj), stride, static_cast<const int*>(positions),
                          static_cast<const int*>(slot_mapping), static_cast<const float*>(table), pairs, table_rows,
                          halves, static_cast<E*>(k_cache), static_cast<E*>(v_cache), QH, KH, VH, D, V, bs,
                          static_cast<const float*>(q_norm), static_cast<const float*>(k_norm), eps));
  return PK_CHECK_LAUNCH();
}

// proj [T, Q | R | Dr]; cq [T, Q] (null with Q = 0); cache rows [slots, R + Dr]
PK_EXPORT int pkm_latent_in(void* cq, void* cache, const void* proj, long long stride, int Q, int R, int Dr, const void* wq,
                            const void* wkv, float eps, const void* positions, const void* slot_mapping,
                            const void* table, int pairs, int table_rows, int halves, int T, int bs, int dt,
                            hipStream_t stream) {
  if (T <= 0) return 0;
  if (R < 1 || Q < 0 || Dr < 0 || 2 * pairs > Dr || (table && table_rows < 1) || (Q > 0 && (!cq || !wq))) return -1;
  const dim3 grid(T, 2);
  PKM_DISPATCH(dt, E, latent_in_kernel<E><<<grid, 256, 0, stream>>>(
                          static_cast<E*>(cq), static_cast<E*>(cache), static_cast<const E*>(proj), stride, Q, R, Dr,
                          static_cast<const float*>(wq), static_cast<const float*>(wkv), eps,
                          static_cast<const int*>(positions), static_cast<const int*>(slot_mapping),
                          static_cast<const float*>(table), pairs, table_rows, halves, bs));
  return PK_CHECK_LAUNCH();
}

// out [T, H, R + Dr]; q_lat [H, T, R]; q [T, H, D + Dr], all of one element type
PK_EXPORT int pkm_latent_query(void* out, const void* q_lat, const void* q, const void* positions, const void* table,
                               int pairs, int table_rows, int halves, int T, int H, int R, int D, int Dr, int dt,
                               hipStream_t stream) {
  if (T <= 0) return 0;
  if (2 * pairs > Dr || (table && table_rows < 1)) return -1;
  const dim3 grid(T, H);
  PKM_DISPATCH(dt, E, latent_query_kernel<E><<<grid, 64, 0, stream>>>(
                          static_cast<E*>(out), static_cast<const E*>(q_lat), static_cast<const E*>(q),
                          static_cast<const int*>(positions), static_cast<const float*>(table), pairs, table_rows, halves,
                          T, H, R, D, Dr));
  return PK_CHECK_LAUNCH();
}

// v_cache == k_cache: the value of a key is the first V numbers of its key row
PK_EXPORT int pkm_masked_attention(void* out, long long out_ts, long long out_hs, int out_dt, const void* q, int q_dt,
                                   const void* k_cache, const void* v_cache, int v_width, const void* block_tables,
                                   long long bt_stride, const void* cu_q, const void* context_lens, const void* sink,
                                   int n_seqs, int T, int QH, int KH, int VH, int D, int V, int bs, float scale, int window,
                                   int chunk, int num_decode, void* ws_o, void* ws_ml, int part, int n_parts, int dt,
                                   hipStream_t stream) {
  if (n_seqs <= 0 || T <= 0) return 0;
  if (KH < 1 || VH < 1 || QH % KH || KH % VH || V < 1 || V > 512 || V > v_width || D < 1) return -1;
  if ((q_dt != dt && q_dt != kF32) || (out_dt != dt && out_dt != kF32)) return -1;
  const bool alias = v_cache == k_cache;
  if (alias && (KH != VH || v_width != D)) return -1;
  const int bk = key_tile(D, V, alias);
  if (bk == 0) return -1;
  MaskedArgs a{out, out_ts, out_hs, out_dt == kF32, q, q_dt == kF32, k_cache, v_cache, v_width,
               static_cast<const int*>(block_tables), bt_stride, static_cast<const int*>(cu_q),
               static_cast<const int*>(context_lens), static_cast<const float*>(sink), n_seqs, QH, KH, VH, D, V, bs, bk,
               scale, window, chunk, 0, 1, nullptr, nullptr};
  const int R = QH / KH;
  if (g_masked_mfma && dt == kBF16 && q_dt == kBF16 && bs % 32 == 0 && v_width % 8 == 0 && mfma_sizes(D, V, alias)) {
    // the first num_decode sequences hold one token each: their bands are cut into runs when a
    // workspace is given (ws_o [num_decode, n_parts, QH, V], ws_ml [num_decode, n_parts, QH, 2] fp32)
    const int nd = (ws_o && ws_ml && n_parts > 1) ? (num_decode < n_seqs ? num_decode : n_seqs) : 0;
    if (nd > 0) {
      if (part < 32 || part % 32 || n_parts > 64) return -1;
      MaskedArgs d = a;
      d.n_seqs = nd;
      d.part = part;
      d.n_parts = n_parts;
      d.ws_o = static_cast<float*>(ws_o);
      d.ws_ml = static_cast<float*>(ws_ml);
      int rc = launch_mfma<true>(d, nd, alias, stream);
      if (rc) return rc;
      masked_merge_kernel<bf16_t><<<dim3(nd, QH), 128, 0, stream>>>(out, out_ts, out_hs, a.out_f32, d.ws_o, d.ws_ml, d.cu_q,
                                                                    d.sink, n_parts, QH, V);
      rc = PK_CHECK_LAUNCH();
      if (rc) return rc;
    }
    if (n_seqs > nd) {
      MaskedArgs p = a;
      p.n_seqs = n_seqs - nd;
      p.block_tables += static_cast<int64_t>(nd) * bt_stride;
      p.cu_q += nd;
      p.context_lens += nd;
      return launch_mfma<false>(p, T - nd, alias, stream);
    }
    return 0;
  }
  // row tiles: every sequence adds at most one partly filled tile
  const int tiles = (T * R + kBQ - 1) / kBQ + n_seqs;
  const dim3 grid(tiles, KH);
  if (alias) {
    PKM_DISPATCH(dt, E, return (launch_masked<E, true>(a, grid, stream)));
  }
  PKM_DISPATCH(dt, E, return (launch_masked<E, false>(a, grid, stream)));
  return 0;
}

// Keys per run of a decoded token's band (a multiple of 32), 0: no split.  `capacity`: the most
// cached tokens of a sequence; the band spans at most window + 31 / chunk + 31 keys from its
// aligned start.  Runs are at least 64 keys, at most 64 of them, and aim at ~512 workgroups per launch.
PK_EXPORT int pkm_masked_decode_part(int nd, int QH, int KH, int D, int V, int alias, int bs, int capacity, int window,
                                     int chunk, int dt) {
  if (!g_masked_mfma || dt != kBF16 || bs % 32 || nd <= 0 || !mfma_sizes(D, V, alias != 0)) return 0;
  int span = capacity;
  if (window > 0 && window + 31 < span) span = window + 31;
  if (chunk > 0 && chunk + 31 < span) span = chunk + 31;
  span = (span + 31) / 32 * 32;
  const int wgs = nd * KH;
  int want = (512 + wgs - 1) / wgs;  // runs wanted
  if (want > 64) want = 64;
  if (want > span / 64) want = span / 64;
  if (want <= 1) return 0;
  return ((span + want - 1) / want + 31) / 32 * 32;
}

PK_EXPORT int pkm_set_masked_mfma(int on) {
  g_masked_mfma = on;
  return 0;
}

// a fp32 [T, H, V] (pair_group = 0) or [T, 2H, V] in groups of (r first maps, r second maps);
// gate [T, H * V] rows gate_stride elements apart (gate_dt) or null; weight fp32 or null, head h reads
// weight[h * weight_hs ...] (0: one [V] for all heads); out rows out_stride elements apart
PK_EXPORT int pkm_head_norm_gate(void* out, long long out_stride, const void* a, int T, int H, int V, float eps,
                                 const void* gate, long long gate_stride, int gate_dt, int gate_kind, const void* weight,
                                 int weight_hs, float post, int pair_group, float coef, int out_dt, hipStream_t stream) {
  if (T <= 0) return 0;
  if (H < 1 || V < 1 || pair_group < 0 || (pair_group > 0 && H % pair_group) || out_stride < static_cast<long long>(H) * V)
    return -1;
  const dim3 grid(T, H);
#define PKM_HNG(GT)                                                                                                  \
  PKM_DISPATCH(out_dt, O, head_norm_gate_kernel<GT, O><<<grid, 64, 0, stream>>>(                                       \
                              static_cast<O*>(out), out_stride, static_cast<const float*>(a), H, V, eps,             \
                              static_cast<const GT*>(gate), gate_stride, gate_kind, static_cast<const float*>(weight),   \
                              weight_hs, post, pair_group, coef))
  if (gate_dt == kF32) {
    PKM_HNG(float);
  } else if (gate_dt == kBF16) {
    PKM_HNG(bf16_t);
  } else {
    return -2;
  }
#undef PKM_HNG
  return PK_CHECK_LAUNCH();
}

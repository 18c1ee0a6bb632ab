// Attention over a sliding window plus pooled blocks behind it, with mixing of the heads'
// softmax weights (gfx950).  Generic sizes, float32 arithmetic, storage T.
//
// A query at position i sees the keys j with 0 <= i - j < size one by one, and for every block
// b of `pool` positions whose last position is behind that window (b*pool + pool - 1 <= i - size) one
// key and one value: the means of the block's cached keys and values.  One softmax per head
// runs over both kinds of entries; the normalised weights of the H heads are then mixed,
//     w'_h(e) = sum_g talk[h, g] w_g(e),
// and head h applies w'_h to the values of its own kv head.
//
// The means live in pages of their own arrays (float32): block b's mean is elements
// [b * W, (b + 1) * W) of the request's flat pooled array, which has ceil(W / pool) elements for
// every position, so a block's mean lies in pages the request already owns when the block is
// complete.  pool_blocks writes the mean of every block that a step completes, summing the
// block's cached rows in position order.
//
// bias_norm_store: the q/k/v projection's output plus biases; q and k each divided by the root
//   mean square of their WHOLE row (all heads) and multiplied by a weight per coordinate; q goes
//   out, k and v into the request's pages.  Page layout: [page][token in page][G * dim].
// pooled_window_attention: a block takes up to TQ consecutive rows of the step (cut where the
//   request changes), walks the entries they see (pooled blocks, then tokens) in chunks staged
//   in LDS, twice: once for every (row, head)'s maximum and sum, once to form the normalised,
//   mixed weights and apply them.
#include "common.h"
#include "slots.h"

using namespace tk;

namespace {

template <typename T>
__device__ __forceinline__ float load_in(const void* p, int f32, int parts, long part_stride, size_t idx) {
  if (!f32) return Elem<T>::load(reinterpret_cast<const T*>(p) + idx);
  const float* f = reinterpret_cast<const float*>(p);
  float s = f[idx];
  for (int i = 1; i < parts; ++i) s += f[idx + (size_t)i * part_stride];
  return s;
}

template <typename T>
__global__ __launch_bounds__(256) void bias_norm_store_kernel(
    const void* __restrict__ qkv, int in_f32, int parts, long part_stride, const float* __restrict__ bias,
    const float* __restrict__ q_weight, const float* __restrict__ k_weight, const int* __restrict__ positions,
    const int* __restrict__ req_of_token, const int* __restrict__ tables, int table_width,
    T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache, int QW, int KW, int VW,
    int page_size, float eps, int store) {
  __shared__ float scratch[16];
  const int n = blockIdx.x;
  const int total = store ? QW + KW + VW : QW;   // a call that only reads the cache projects q alone
  const size_t row = (size_t)n * total;
  float sq = 0.f, sk = 0.f;
  for (int c = threadIdx.x; c < QW; c += blockDim.x) {
    const float x = load_in<T>(qkv, in_f32, parts, part_stride, row + c) + bias[c];
    sq += x * x;
  }
  sq = block_sum(sq, scratch);
  const float rq = 1.f / sqrtf(sq / (float)QW + eps);
  for (int c = threadIdx.x; c < QW; c += blockDim.x) {
    const float x = load_in<T>(qkv, in_f32, parts, part_stride, row + c) + bias[c];
    Elem<T>::store(q_out + (size_t)n * QW + c, x * rq * q_weight[c]);
  }
  if (!store) return;
  for (int c = threadIdx.x; c < KW; c += blockDim.x) {
    const float x = load_in<T>(qkv, in_f32, parts, part_stride, row + QW + c) + bias[QW + c];
    sk += x * x;
  }
  sk = block_sum(sk, scratch);
  const float rk = 1.f / sqrtf(sk / (float)KW + eps);
  const int pos = positions[n];
  const int page = tables[(size_t)req_of_token[n] * table_width + pos / page_size];
  const size_t slot = (size_t)page * page_size + pos % page_size;
  for (int c = threadIdx.x; c < KW; c += blockDim.x) {
    const float x = load_in<T>(qkv, in_f32, parts, part_stride, row + QW + c) + bias[QW + c];
    Elem<T>::store(k_cache + slot * KW + c, x * rk * k_weight[c]);
  }
  for (int c = threadIdx.x; c < VW; c += blockDim.x) {
    const float x = load_in<T>(qkv, in_f32, parts, part_stride, row + QW + KW + c) + bias[QW + KW + c];
    Elem<T>::store(v_cache + slot * VW + c, x);
  }
}

// element c of block b's mean in a pooled array with E elements a position
__device__ __forceinline__ size_t pooled_at(const int* __restrict__ table, int b, int c, int width, int E,
                                            int page_size) {
  const size_t flat = (size_t)b * width + c;
  const size_t per_page = (size_t)page_size * E;
  return (size_t)table[flat / per_page] * per_page + flat % per_page;
}

// a token that completes a block of `pool` positions writes the block's mean key and value
template <typename T>
__global__ __launch_bounds__(256) void pool_blocks_kernel(
    const T* __restrict__ k_cache, const T* __restrict__ v_cache, float* __restrict__ k_pool,
    float* __restrict__ v_pool, const int* __restrict__ positions, const int* __restrict__ req_of_token,
    const int* __restrict__ tables, int table_width, int KW, int VW, int KE, int VE, int pool, int page_size) {
  const int n = blockIdx.x;
  const int pos = positions[n];
  if ((pos + 1) % pool != 0) return;
  const int b = pos / pool;
  const int* table = tables + (size_t)req_of_token[n] * table_width;
  const float inv = 1.f / (float)pool;
  for (int c = threadIdx.x; c < KW + VW; c += blockDim.x) {
    const bool key = c < KW;
    const int width = key ? KW : VW, col = key ? c : c - KW;
    const T* cache = key ? k_cache : v_cache;
    float s = 0.f;
    for (int t = 0; t < pool; ++t) {
      const int p = b * pool + t;
      s += Elem<T>::load(cache + ((size_t)table[p / page_size] * page_size + p % page_size) * width + col);
    }
    if (key) k_pool[pooled_at(table, b, col, KW, KE, page_size)] = s * inv;
    else v_pool[pooled_at(table, b, col, VW, VE, page_size)] = s * inv;
  }
}

// The same for rows of up to 8 * 1024 numbers: a thread holds its eight in registers, so every
// load of the row is asked for at once and the row is read once.
constexpr int kRowRegs = 8;
template <typename T>
__global__ __launch_bounds__(1024) void bias_norm_store_row_kernel(
    const void* __restrict__ qkv, int in_f32, int parts, long part_stride, const float* __restrict__ bias,
    const float* __restrict__ q_weight, const float* __restrict__ k_weight, const int* __restrict__ positions,
    const int* __restrict__ req_of_token, const int* __restrict__ tables, int table_width,
    T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache, int QW, int KW, int VW,
    int page_size, float eps, int store) {
  __shared__ float scratch[16];
  const int n = blockIdx.x;
  const int total = store ? QW + KW + VW : QW;
  const size_t row = (size_t)n * total;
  float x[kRowRegs];
#pragma unroll
  for (int u = 0; u < kRowRegs; ++u) {
    const int c = threadIdx.x + u * blockDim.x;
    x[u] = c < total ? bias[c] : 0.f;
  }
  if (!in_f32) {
#pragma unroll
    for (int u = 0; u < kRowRegs; ++u) {
      const int c = threadIdx.x + u * blockDim.x;
      if (c < total) x[u] += Elem<T>::load(reinterpret_cast<const T*>(qkv) + row + c);
    }
  } else {
    // partial sums of a split product: four parts' loads asked for together, added in the parts' order
    const float* f = reinterpret_cast<const float*>(qkv) + row;
    int i = 0;
    for (; i + 3 < parts; i += 4) {
      float y[4][kRowRegs];
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int u = 0; u < kRowRegs; ++u) {
          const int c = threadIdx.x + u * blockDim.x;
          y[j][u] = c < total ? f[c + (size_t)(i + j) * part_stride] : 0.f;
        }
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int u = 0; u < kRowRegs; ++u) x[u] += y[j][u];
    }
    for (; i < parts; ++i) {
#pragma unroll
      for (int u = 0; u < kRowRegs; ++u) {
        const int c = threadIdx.x + u * blockDim.x;
        if (c < total) x[u] += f[c + (size_t)i * part_stride];
      }
    }
  }
  float sq = 0.f, sk = 0.f;
#pragma unroll
  for (int u = 0; u < kRowRegs; ++u) {
    const int c = threadIdx.x + u * blockDim.x;
    if (c < QW) sq += x[u] * x[u];
    else if (c < QW + KW) sk += x[u] * x[u];
  }
  sq = block_sum(sq, scratch);
  if (store) sk = block_sum(sk, scratch);
  const float rq = 1.f / sqrtf(sq / (float)QW + eps), rk = 1.f / sqrtf(sk / (float)KW + eps);
  size_t slot = 0;
  if (store) {
    const int pos = positions[n];
    slot = (size_t)tables[(size_t)req_of_token[n] * table_width + pos / page_size] * page_size + pos % page_size;
  }
#pragma unroll
  for (int u = 0; u < kRowRegs; ++u) {
    const int c = threadIdx.x + u * blockDim.x;
    if (c < QW) Elem<T>::store(q_out + (size_t)n * QW + c, x[u] * rq * q_weight[c]);
    else if (c < QW + KW) Elem<T>::store(k_cache + slot * KW + (c - QW), x[u] * rk * k_weight[c - QW]);
    else if (c < total) Elem<T>::store(v_cache + slot * VW + (c - QW - KW), x[u]);
  }
}

struct PoolArgs {
  const int* positions;
  const int* req_of_token;
  const int* q_start;
  const int* tables;
  const float* talk;
  const float* k_pool;
  const float* v_pool;
  int table_width, N, H, G, dim, vdim, size, pool, page_size, TQ, CH, KE, VE;
  float scale;
};

constexpr int kAcc = 16;   // outputs a thread accumulates: TQ * H * vdim <= kAcc * blockDim

// rows [e0, e0 + ne) of a chunk: entry e < NB is block e's mean, else token j0 + (e - NB)
template <typename T>
__device__ __forceinline__ void stage(const T* __restrict__ cache, const float* __restrict__ pooled,
                                      const int* __restrict__ table, float* dst, int width, int padded, int e0,
                                      int ne, int NB, int j0, int E, int page_size) {
  for (int idx = threadIdx.x; idx < ne * width; idx += blockDim.x) {
    const int e = idx / width, c = idx - e * width;
    const int entry = e0 + e;
    float v;
    if (entry < NB) {
      v = pooled[pooled_at(table, entry, c, width, E, page_size)];
    } else {
      const int p = j0 + entry - NB;
      v = Elem<T>::load(cache + ((size_t)table[p / page_size] * page_size + p % page_size) * width + c);
    }
    dst[e * padded + c] = v;
  }
}

template <typename T>
__global__ void pooled_window_attention_kernel(const T* __restrict__ q, const T* __restrict__ k_cache,
                                               const T* __restrict__ v_cache, T* __restrict__ out, PoolArgs a) {
  extern __shared__ float lds[];
  const int H = a.H, G = a.G, dim = a.dim, vdim = a.vdim, CH = a.CH, TQ = a.TQ;
  const int QW = H * dim, KW = G * dim, VW = G * vdim, KP = KW + 1, VP = VW + 1;
  const int group = H / G;
  float* qs = lds;                       // [TQ][QW]
  float* Ks = qs + TQ * QW;              // [CH][KP]
  float* Vs = Ks + CH * KP;              // [CH][VP]
  float* sc = Vs + CH * VP;              // [TQ][H][CH]
  float* wm = sc + TQ * H * CH;          // [TQ][H][CH]
  float* mx = wm + TQ * H * CH;          // [TQ][H]
  float* sm = mx + TQ * H;               // [TQ][H]
  float* tk_ = sm + TQ * H;              // [H][H]
  const int tid = threadIdx.x, nthreads = blockDim.x;
  const int lane = tid & (kWave - 1), wave = tid / kWave, nwaves = nthreads / kWave;
  for (int i = tid; i < H * H; i += nthreads) tk_[i] = a.talk[i];

  const int row_end = min(a.N, (int)(blockIdx.x + 1) * TQ);
  int row = blockIdx.x * TQ;
  while (row < row_end) {
    const int r = a.req_of_token[row];
    const int seg_end = min(row_end, a.q_start[r + 1]);
    const int tq = seg_end - row;
    const int i0 = a.positions[row], i_last = i0 + tq - 1;
    const int* table = a.tables + (size_t)r * a.table_width;
    const int behind = i_last - a.size - (a.pool - 1);
    const int NB = behind >= 0 ? behind / a.pool + 1 : 0;
    const int j0 = max(0, i0 - a.size + 1);
    const int E = NB + i_last - j0 + 1;

    __syncthreads();   // the segment before is done with the shared arrays
    for (int i = tid; i < tq * QW; i += nthreads) qs[i] = Elem<T>::load(q + (size_t)row * QW + i);
    for (int i = tid; i < tq * H; i += nthreads) {
      mx[i] = -INFINITY;
      sm[i] = 0.f;
    }

    for (int pass = 0; pass < 2; ++pass) {
      float acc[kAcc];
#pragma unroll
      for (int x = 0; x < kAcc; ++x) acc[x] = 0.f;
      for (int e0 = 0; e0 < E; e0 += CH) {
        const int ne = min(CH, E - e0);
        __syncthreads();
        stage<T>(k_cache, a.k_pool, table, Ks, KW, KP, e0, ne, NB, j0, a.KE, a.page_size);
        if (pass == 1) stage<T>(v_cache, a.v_pool, table, Vs, VW, VP, e0, ne, NB, j0, a.VE, a.page_size);
        __syncthreads();
        // scores, or (second pass) normalised weights
        for (int idx = tid; idx < tq * H * ne; idx += nthreads) {
          const int e = idx % ne, th = idx / ne, g = th % H, t = th / H;
          const int i = i0 + t, entry = e0 + e;
          bool seen;
          if (entry < NB) {
            seen = entry * a.pool + a.pool - 1 <= i - a.size;
          } else {
            const int j = j0 + entry - NB;
            seen = j <= i && i - j < a.size;
          }
          float s = -INFINITY;
          if (seen) {
            const float* qv = qs + t * QW + g * dim;
            const float* kv = Ks + e * KP + (g / group) * dim;
            float d = 0.f;
            for (int x = 0; x < dim; ++x) d = fmaf(qv[x], kv[x], d);
            s = d * a.scale;
          }
          if (pass == 1) s = seen ? expf(s - mx[th]) / sm[th] : 0.f;
          sc[th * CH + e] = s;
        }
        __syncthreads();
        if (pass == 0) {
          // running maximum and sum of every (row, head), a wave each
          for (int th = wave; th < tq * H; th += nwaves) {
            float m = -INFINITY;
            for (int e = lane; e < ne; e += kWave) m = fmaxf(m, sc[th * CH + e]);
            m = wave_max(m);
            const float m_old = mx[th];
            const float m_new = fmaxf(m_old, m);
            if (m_new > -INFINITY) {
              float s = 0.f;
              for (int e = lane; e < ne; e += kWave) {
                const float v = sc[th * CH + e];
                if (v > -INFINITY) s += expf(v - m_new);
              }
              s = wave_sum(s);
              if (lane == 0) {
                sm[th] = (m_old > -INFINITY ? sm[th] * expf(m_old - m_new) : 0.f) + s;
                mx[th] = m_new;
              }
            }
          }
        } else {
          for (int idx = tid; idx < tq * H * ne; idx += nthreads) {
            const int e = idx % ne, th = idx / ne, h = th % H, t = th / H;
            float w = 0.f;
            for (int g = 0; g < H; ++g) w = fmaf(tk_[h * H + g], sc[(t * H + g) * CH + e], w);
            wm[th * CH + e] = w;
          }
          __syncthreads();
#pragma unroll
          for (int x = 0; x < kAcc; ++x) {
            const int o = tid + x * nthreads;
            if (o < tq * H * vdim) {
              const int d = o % vdim, th = o / vdim, h = th % H;
              const float* w = wm + th * CH;
              const float* v = Vs + (h / group) * vdim + d;
              float s = acc[x];
              for (int e = 0; e < ne; ++e) s = fmaf(w[e], v[e * VP], s);
              acc[x] = s;
            }
          }
        }
      }
      if (pass == 1) {
#pragma unroll
        for (int x = 0; x < kAcc; ++x) {
          const int o = tid + x * nthreads;
          if (o < tq * H * vdim) Elem<T>::store(out + (size_t)row * H * vdim + o, acc[x]);
        }
      }
    }
    row = seg_end;
  }
}


// ---------------------------------------------------------------------------
// The same attention in four kernels that fill the GPU whatever the step's shape: a block
// takes up to TQ consecutive rows of one request, ONE kv head and one share of the entries.
//   scores:  a lane an entry: its key row (or block mean) against the queries of the kv head's
//            query heads; raw scores to memory [row][entry][head], and every (row, head)'s
//            maximum and sum of exponentials over the share.
//   normalize: merges the shares' statistics, turns the scores of ALL heads into normalised
//            weights and mixes them, in place (each exponential and each mixed weight once).
//   values:  applies the mixed weights of its own query heads to its
//            kv head's values (64 entries staged in LDS at a time; a thread owns four channels of a few
//            (row, head) pairs); float32 partial outputs.
//   merge:   adds the shares' partial outputs.
constexpr int kGroupMax = 16;   // query heads a kv head
constexpr int kTileMax = 8;     // rows a block
constexpr int kPairMax = 32;    // rows times query heads a lane accumulates in the score kernel
constexpr int kSplitThreads = 256;

struct SplitArgs {
  const int* positions;
  const int* req_of_token;
  const int* q_start;
  const int* tables;
  const float* talk;
  const float* k_pool;
  const float* v_pool;
  float* scores;     // [N][Emax][H]
  float* part_m;     // [N][H][S]
  float* part_l;     // [N][H][S]
  float* part_o;     // [S][N][H * vdim]
  int table_width, N, H, G, dim, vdim, size, pool, page_size, TQ, S, Emax, KE, VE;
  float scale;
};

struct Segment {
  int row, tq, i0, NB, j0, E;
  const int* table;
};

// the rows [row, seg_end) of one request inside a block's tile, and the entries they see together
__device__ __forceinline__ Segment segment_at(const SplitArgs& a, int row, int row_end) {
  Segment g;
  const int r = a.req_of_token[row];
  g.row = row;
  g.tq = min(row_end, a.q_start[r + 1]) - row;
  g.i0 = a.positions[row];
  const int i_last = g.i0 + g.tq - 1;
  const int behind = i_last - a.size - (a.pool - 1);
  g.NB = behind >= 0 ? behind / a.pool + 1 : 0;
  g.j0 = max(0, g.i0 - a.size + 1);
  g.E = g.NB + i_last - g.j0 + 1;
  g.table = a.tables + (size_t)r * a.table_width;
  return g;
}

__device__ __forceinline__ bool entry_seen(const SplitArgs& a, const Segment& g, int entry, int i) {
  if (entry < g.NB) return entry * a.pool + a.pool - 1 <= i - a.size;
  const int j = g.j0 + entry - g.NB;
  return j <= i && i - j < a.size;
}

template <typename T>
__device__ __forceinline__ float entry_value(const T* __restrict__ cache, const float* __restrict__ pooled,
                                             const Segment& g, int entry, int col, int width, int E, int page_size) {
  if (entry < g.NB) return pooled[pooled_at(g.table, entry, col, width, E, page_size)];
  const int p = g.j0 + entry - g.NB;
  return Elem<T>::load(cache + ((size_t)g.table[p / page_size] * page_size + p % page_size) * width + col);
}

__device__ __forceinline__ void load8(const float* p, float* o) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w;
  o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
}
__device__ __forceinline__ void load8(const bf16_t* p, float* o) {
  const uint4 v = *reinterpret_cast<const uint4*>(p);
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    o[2 * i] = __uint_as_float(w[i] << 16);
    o[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}

template <typename T>
__global__ __launch_bounds__(kSplitThreads) void pooled_scores_kernel(const T* __restrict__ q,
                                                                      const T* __restrict__ k_cache, SplitArgs a) {
  extern __shared__ float lds[];
  const int group = a.H / a.G, dim = a.dim, KW = a.G * a.dim;
  const int c = blockIdx.y, split = blockIdx.z;
  float* qs = lds;                                   // [TQ][group][dim]
  float* red = qs + a.TQ * group * dim;              // [waves][TQ * group][2]
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  constexpr int kWaves = kSplitThreads / kWave;
  const int row_end = min(a.N, (int)(blockIdx.x + 1) * a.TQ);
  int row = blockIdx.x * a.TQ;
  while (row < row_end) {
    const Segment g = segment_at(a, row, row_end);
    const int pairs = g.tq * group;
    __syncthreads();
    for (int i = tid; i < pairs * dim; i += kSplitThreads) {
      const int x = i % dim, tg = i / dim, t = tg / group, h = tg % group;
      qs[i] = Elem<T>::load(q + (size_t)(g.row + t) * a.H * dim + (c * group + h) * dim + x);
    }
    __syncthreads();
    const int e_lo = (int)((long)g.E * split / a.S), e_hi = (int)((long)g.E * (split + 1) / a.S);
    // 16-byte loads where every row starts on a 16-byte border
    const bool vec = dim % 8 == 0 && KW % 8 == 0;
    const bool pvec = vec && ((long)a.page_size * a.KE) % 4 == 0;
    float m[kPairMax], l[kPairMax];
#pragma unroll
    for (int p = 0; p < kPairMax; ++p) {
      m[p] = -INFINITY;
      l[p] = 0.f;
    }
    for (int entry = e_lo + tid; entry < e_hi; entry += kSplitThreads) {
      float acc[kPairMax];
#pragma unroll
      for (int p = 0; p < kPairMax; ++p) acc[p] = 0.f;
      // the entry's row for this kv head: a cache row, a block mean inside one page, or (a mean
      // across a page border) neither, and then element by element
      const T* rowp = nullptr;
      const float* poolp = nullptr;
      if (entry < g.NB) {
        const size_t first = (size_t)entry * KW + (size_t)c * dim, per_page = (size_t)a.page_size * a.KE;
        if (first % per_page + dim <= per_page) poolp = a.k_pool + (size_t)g.table[first / per_page] * per_page + first % per_page;
      } else {
        const int p = g.j0 + entry - g.NB;
        rowp = k_cache + ((size_t)g.table[p / a.page_size] * a.page_size + p % a.page_size) * KW + (size_t)c * dim;
      }
      if ((rowp != nullptr && vec) || (poolp != nullptr && pvec)) {
        // 64 elements of the row asked for at once (eight 16- or 32-byte loads in flight), then
        // the products, the queries read from LDS four at a time
        for (int x0 = 0; x0 < dim; x0 += 64) {
          float kx[64];
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            if (x0 + 8 * u < dim) {
              if (rowp != nullptr) load8(rowp + x0 + 8 * u, kx + 8 * u);
              else load8(poolp + x0 + 8 * u, kx + 8 * u);
            }
          }
#pragma unroll
          for (int u = 0; u < 16; ++u) {
            if (x0 + 4 * u < dim) {
#pragma unroll
              for (int p = 0; p < kPairMax; ++p) {
                if (p < pairs) {
                  const float4 qv = *reinterpret_cast<const float4*>(qs + p * dim + x0 + 4 * u);
                  acc[p] = fmaf(qv.x, kx[4 * u], fmaf(qv.y, kx[4 * u + 1], fmaf(qv.z, kx[4 * u + 2], fmaf(qv.w, kx[4 * u + 3], acc[p]))));
                }
              }
            }
          }
        }
      } else {
        for (int x = 0; x < dim; ++x) {
          const float kx = rowp != nullptr ? Elem<T>::load(rowp + x)
                           : poolp != nullptr ? poolp[x]
                                              : entry_value<T>(k_cache, a.k_pool, g, entry, c * dim + x, KW, a.KE, a.page_size);
#pragma unroll
          for (int p = 0; p < kPairMax; ++p)
            if (p < pairs) acc[p] = fmaf(qs[p * dim + x], kx, acc[p]);
        }
      }
#pragma unroll
      for (int p = 0; p < kPairMax; ++p) {
        if (p < pairs) {
          const int t = p / group, h = p % group;
          const bool seen = entry_seen(a, g, entry, g.i0 + t);
          const float sc = seen ? acc[p] * a.scale : -INFINITY;
          a.scores[((size_t)(g.row + t) * a.Emax + entry) * a.H + c * group + h] = sc;
          if (seen) {
            const float m_new = fmaxf(m[p], sc);
            l[p] = l[p] * expf(m[p] - m_new) + expf(sc - m_new);     // (exp(-inf) = 0 the first time)
            m[p] = m_new;
          }
        }
      }
    }
    // the block's maximum and sum of every (row, head): lanes, then waves
#pragma unroll
    for (int p = 0; p < kPairMax; ++p) {
      if (p < pairs) {
        const float m_all = wave_max(m[p]);
        const float l_all = wave_sum(m[p] > -INFINITY ? l[p] * expf(m[p] - m_all) : 0.f);
        if (lane == 0) {
          red[(wave * kPairMax + p) * 2] = m_all;
          red[(wave * kPairMax + p) * 2 + 1] = l_all;
        }
      }
    }
    __syncthreads();
    for (int p = tid; p < pairs; p += kSplitThreads) {
      float m_all = -INFINITY;
      for (int w = 0; w < kWaves; ++w) m_all = fmaxf(m_all, red[(w * kPairMax + p) * 2]);
      float l_all = 0.f;
      for (int w = 0; w < kWaves; ++w) {
        const float mw = red[(w * kPairMax + p) * 2];
        if (mw > -INFINITY) l_all += red[(w * kPairMax + p) * 2 + 1] * expf(mw - m_all);
      }
      const int t = p / group, h = p % group;
      const size_t at = ((size_t)(g.row + t) * a.H + c * group + h) * a.S + split;
      a.part_m[at] = m_all;
      a.part_l[at] = l_all;
    }
    row += g.tq;
  }
}

// The score kernel on the matrix cores (bfloat16 storage, dim a multiple of 16, rows on 16-byte
// borders).  A wave takes 32 token entries at a time: S^T[entry][pair] = K[entry][:] . Q[pair][:]
// with v_mfma_f32_32x32x16_bf16, A = 32 key rows x 16 channels straight from the pages (lane
// (col, g) loads channels [16 c + 8 g, + 8) of entry col's row), B = the tile's queries, kept in
// registers for the whole walk (pair col = row * group + head; pairs beyond the tile's are
// zero).  A lane then holds, for its pair, the entries 8 i + 4 g + j (i, j < 4) of the 32.  The
// products of bfloat16 numbers are exact in float32 and are added in float32.  The few block
// means (float32) keep the vector path above, by the same lanes, before the tokens.
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));
union KeyFrag {
  uint4 u;
  bf16x8_t v;
};
constexpr int kStepsMax = 16;   // 16-channel steps: dim <= 256

__global__ __launch_bounds__(kSplitThreads) void pooled_scores_mfma_kernel(const bf16_t* __restrict__ q,
                                                                           const bf16_t* __restrict__ k_cache,
                                                                           SplitArgs a) {
  extern __shared__ float lds[];
  const int group = a.H / a.G, dim = a.dim, KW = a.G * a.dim, steps = dim / 16;
  const int c = blockIdx.y, split = blockIdx.z;
  float* qs = lds;                                   // [TQ][group][dim] (for the block means)
  float* red = qs + a.TQ * group * dim;              // [2 waves' worth][kPairMax][2]
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  constexpr int kWaves = kSplitThreads / kWave;
  const int col = lane & 31, g = lane >> 5;
  const int row_end = min(a.N, (int)(blockIdx.x + 1) * a.TQ);
  int row = blockIdx.x * a.TQ;
  while (row < row_end) {
    const Segment sg = segment_at(a, row, row_end);
    const int pairs = sg.tq * group;
    __syncthreads();
    for (int i = tid; i < pairs * dim; i += kSplitThreads) {
      const int x = i % dim, tg = i / dim, t = tg / group, h = tg % group;
      qs[i] = Elem<bf16_t>::load(q + (size_t)(sg.row + t) * a.H * dim + (c * group + h) * dim + x);
    }
    // this lane's pair and its query fragments
    const bool pair_live = col < pairs;
    const int my_t = col / group, my_h = col % group;
    const int my_i = sg.i0 + my_t;
    KeyFrag qreg[kStepsMax];
#pragma unroll
    for (int s = 0; s < kStepsMax; ++s) {
      qreg[s].u = make_uint4(0, 0, 0, 0);
      if (s < steps && pair_live)
        qreg[s].u = *reinterpret_cast<const uint4*>(q + (size_t)(sg.row + my_t) * a.H * dim + (c * group + my_h) * dim +
                                                    16 * s + 8 * g);
    }
    __syncthreads();
    const int e_lo = (int)((long)sg.E * split / a.S), e_hi = (int)((long)sg.E * (split + 1) / a.S);
    // --- block means: a lane an entry, every pair (few entries; float32 throughout) ---
    float m[kPairMax], l[kPairMax];
#pragma unroll
    for (int p = 0; p < kPairMax; ++p) {
      m[p] = -INFINITY;
      l[p] = 0.f;
    }
    const int pooled_hi = min(e_hi, sg.NB);
    for (int entry = e_lo + tid; entry < pooled_hi; entry += kSplitThreads) {
      float acc[kPairMax];
#pragma unroll
      for (int p = 0; p < kPairMax; ++p) acc[p] = 0.f;
      const size_t first = (size_t)entry * KW + (size_t)c * dim, per_page = (size_t)a.page_size * a.KE;
      if (per_page % 4 == 0 && first % per_page + dim <= per_page) {
        // the mean lies in one page, on a 32-byte border (dim and KW are multiples of 16): 64 numbers asked for at once
        const float* poolp = a.k_pool + (size_t)sg.table[first / per_page] * per_page + first % per_page;
        for (int x0 = 0; x0 < dim; x0 += 64) {
          float kx[64];
#pragma unroll
          for (int u = 0; u < 8; ++u)
            if (x0 + 8 * u < dim) load8(poolp + x0 + 8 * u, kx + 8 * u);
#pragma unroll
          for (int u = 0; u < 16; ++u) {
            if (x0 + 4 * u < dim) {
#pragma unroll
              for (int p = 0; p < kPairMax; ++p) {
                if (p < pairs) {
                  const float4 qv = *reinterpret_cast<const float4*>(qs + p * dim + x0 + 4 * u);
                  acc[p] = fmaf(qv.x, kx[4 * u], fmaf(qv.y, kx[4 * u + 1], fmaf(qv.z, kx[4 * u + 2], fmaf(qv.w, kx[4 * u + 3], acc[p]))));
                }
              }
            }
          }
        }
      } else {
        for (int x = 0; x < dim; ++x) {
          const float kx = a.k_pool[pooled_at(sg.table, entry, c * dim + x, KW, a.KE, a.page_size)];
#pragma unroll
          for (int p = 0; p < kPairMax; ++p)
            if (p < pairs) acc[p] = fmaf(qs[p * dim + x], kx, acc[p]);
        }
      }
#pragma unroll
      for (int p = 0; p < kPairMax; ++p) {
        if (p < pairs) {
          const int t = p / group, h = p % group;
          const bool seen = entry_seen(a, sg, entry, sg.i0 + t);
          const float sc = seen ? acc[p] * a.scale : -INFINITY;
          a.scores[((size_t)(sg.row + t) * a.Emax + entry) * a.H + c * group + h] = sc;
          if (seen) {
            const float m_new = fmaxf(m[p], sc);
            l[p] = l[p] * expf(m[p] - m_new) + expf(sc - m_new);
            m[p] = m_new;
          }
        }
      }
    }
#pragma unroll
    for (int p = 0; p < kPairMax; ++p) {
      if (p < pairs) {
        const float m_all = wave_max(m[p]);
        const float l_all = wave_sum(m[p] > -INFINITY ? l[p] * expf(m[p] - m_all) : 0.f);
        if (lane == 0) {
          red[(wave * kPairMax + p) * 2] = m_all;
          red[(wave * kPairMax + p) * 2 + 1] = l_all;
        }
      }
    }
    // --- tokens: 32 entries a wave and turn, on the matrix cores ---
    const int t_lo = max(e_lo, sg.NB);
    float mm = -INFINITY, ll = 0.f;      // of this lane's pair over the entries it holds
    for (int e0 = t_lo + 32 * wave; e0 < e_hi; e0 += 32 * kWaves) {
      const int mine = min(e0 + col, e_hi - 1);       // (a row that exists; what lies past the share is not used)
      const int pos = sg.j0 + mine - sg.NB;
      const bf16_t* rowp = k_cache + ((size_t)sg.table[pos / a.page_size] * a.page_size + pos % a.page_size) * KW +
                           (size_t)c * dim + 8 * g;
      KeyFrag kf[kStepsMax];
#pragma unroll
      for (int s = 0; s < kStepsMax; ++s)
        if (s < steps) kf[s].u = *reinterpret_cast<const uint4*>(rowp + 16 * s);
      float16_t acc;
#pragma unroll
      for (int x = 0; x < 16; ++x) acc[x] = 0.f;
#pragma unroll
      for (int s = 0; s < kStepsMax; ++s)
        if (s < steps) acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[s].v, qreg[s].v, acc, 0, 0, 0);
      if (pair_live) {
#pragma unroll
        for (int x = 0; x < 16; ++x) {
          const int entry = e0 + 8 * (x >> 2) + 4 * g + (x & 3);
          if (entry < e_hi) {
            const int j = sg.j0 + entry - sg.NB;
            const bool seen = j <= my_i && my_i - j < a.size;
            const float sc = seen ? acc[x] * a.scale : -INFINITY;
            a.scores[((size_t)(sg.row + my_t) * a.Emax + entry) * a.H + c * group + my_h] = sc;
            if (seen) {
              const float m_new = fmaxf(mm, sc);
              ll = ll * expf(mm - m_new) + expf(sc - m_new);
              mm = m_new;
            }
          }
        }
      }
    }
    {   // the two halves of the wave hold the same pairs
      const float m_other = __shfl_xor(mm, 32, kWave), l_other = __shfl_xor(ll, 32, kWave);
      const float m_all = fmaxf(mm, m_other);
      const float l_all = (mm > -INFINITY ? ll * expf(mm - m_all) : 0.f) + (m_other > -INFINITY ? l_other * expf(m_other - m_all) : 0.f);
      if (g == 0 && pair_live) {
        red[((kWaves + wave) * kPairMax + col) * 2] = m_all;
        red[((kWaves + wave) * kPairMax + col) * 2 + 1] = l_all;
      }
    }
    __syncthreads();
    for (int p = tid; p < pairs; p += kSplitThreads) {
      float m_all = -INFINITY;
      for (int w = 0; w < 2 * kWaves; ++w) m_all = fmaxf(m_all, red[(w * kPairMax + p) * 2]);
      float l_all = 0.f;
      for (int w = 0; w < 2 * kWaves; ++w) {
        const float mw = red[(w * kPairMax + p) * 2];
        if (mw > -INFINITY) l_all += red[(w * kPairMax + p) * 2 + 1] * expf(mw - m_all);
      }
      const int t = p / group, h = p % group;
      const size_t at = ((size_t)(sg.row + t) * a.H + c * group + h) * a.S + split;
      a.part_m[at] = m_all;
      a.part_l[at] = l_all;
    }
    row += sg.tq;
  }
}

// scores -> normalised and MIXED weights, in place, for all heads of a row: a block a (row, 256
// entries), a thread an entry.  The shares' maxima and sums of the row's heads are loaded side by
// side and merged in LDS first; then w_g = exp(s_g - max_g) / sum_g for every head in registers and
// w'_h = sum_g talk[h, g] w_g written over the scores.  Each exponential and each mixed weight is
// formed once here, and a kv head's value kernel reads its own heads' weights only.
constexpr int kHeadsMax = 64;
__global__ __launch_bounds__(kSplitThreads) void pooled_normalize_kernel(SplitArgs a) {
  extern __shared__ float lds[];
  const int H = a.H, S = a.S;
  const int Hp = (H + 3) & ~3;
  float* tkk = lds;                 // [H][Hp] the mixing matrix, rows padded to four with zeros
  float* sm_ = tkk + H * Hp;        // [H][S] maxima, then as many sums
  float* mh = sm_ + 2 * H * S;      // [H]
  float* il = mh + H;               // [H]
  const int row = blockIdx.x, tid = threadIdx.x;
  const int count = H * S;
  const size_t from = (size_t)row * count;
  for (int i = tid; i < H * Hp; i += kSplitThreads) tkk[i] = i % Hp < H ? a.talk[(i / Hp) * H + i % Hp] : 0.f;
  for (int i = tid; i < count; i += kSplitThreads) {
    sm_[i] = a.part_m[from + i];
    sm_[count + i] = a.part_l[from + i];
  }
  __syncthreads();
  for (int h = tid; h < H; h += kSplitThreads) {
    float m_all = -INFINITY;
    for (int sh = 0; sh < S; ++sh) m_all = fmaxf(m_all, sm_[h * S + sh]);
    float l_all = 0.f;
    for (int sh = 0; sh < S; ++sh) {
      const float ms = sm_[h * S + sh];
      if (ms > -INFINITY) l_all += sm_[count + h * S + sh] * expf(ms - m_all);
    }
    mh[h] = m_all;
    il[h] = 1.f / l_all;
  }
  __syncthreads();
  // the entries of the row's segment (the rows of its request inside its tile), as the score kernel numbers them
  const int r = a.req_of_token[row];
  const int tile = row / a.TQ * a.TQ;
  const int seg_start = max(tile, a.q_start[r]), seg_end = min(min(a.N, tile + a.TQ), a.q_start[r + 1]);
  const int i0 = a.positions[row] - (row - seg_start), i_last = a.positions[row] + (seg_end - 1 - row);
  const int behind = i_last - a.size - (a.pool - 1);
  const int E = (behind >= 0 ? behind / a.pool + 1 : 0) + i_last - max(0, i0 - a.size + 1) + 1;
  const int e = blockIdx.y * kSplitThreads + tid;
  if (e >= E) return;
  float* sc = a.scores + ((size_t)row * a.Emax + e) * H;
  // the entry's normalised weights of every head, in registers
  float w[kHeadsMax];
#pragma unroll
  for (int g4 = 0; g4 < kHeadsMax; g4 += 4) {
    if (g4 < H) {
      float v[4];
      if (H % 4 == 0) {
        const float4 f = *reinterpret_cast<const float4*>(sc + g4);
        v[0] = f.x; v[1] = f.y; v[2] = f.z; v[3] = f.w;
      } else {
#pragma unroll
        for (int y = 0; y < 4; ++y) v[y] = g4 + y < H ? sc[g4 + y] : -INFINITY;
      }
#pragma unroll
      for (int y = 0; y < 4; ++y)
        w[g4 + y] = (g4 + y < H && v[y] > -INFINITY) ? expf(v[y] - mh[g4 + y]) * il[g4 + y] : 0.f;
    } else {
#pragma unroll
      for (int y = 0; y < 4; ++y) w[g4 + y] = 0.f;
    }
  }
  // mixed: w'_h = sum_g talk[h, g] w_g, written over the scores
  for (int h = 0; h < H; ++h) {
    const float* trow = tkk + h * Hp;
    float acc = 0.f;
#pragma unroll
    for (int g4 = 0; g4 < kHeadsMax; g4 += 4) {
      if (g4 < H) {
        const float4 t4 = *reinterpret_cast<const float4*>(trow + g4);     // (rows padded with zeros to four)
        acc = fmaf(t4.x, w[g4], fmaf(t4.y, w[g4 + 1], fmaf(t4.z, w[g4 + 2], fmaf(t4.w, w[g4 + 3], acc))));
      }
    }
    sc[h] = acc;
  }
}

constexpr int kStage = 64;     // entries whose values are staged in LDS at once
constexpr int kOwnMax = 8;     // (row, head) pairs a thread of the value kernel owns

__device__ __forceinline__ float4 load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 load4(const bf16_t* p) {
  const uint2 v = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u), __uint_as_float(v.y << 16),
                     __uint_as_float(v.y & 0xffff0000u));
}

// four channels from column `col` on (the first `valid` exist) of an entry's value row
template <typename T>
__device__ __forceinline__ float4 load_unit(const T* __restrict__ cache, const float* __restrict__ pooled,
                                            const Segment& g, int entry, int col, int valid, int width, int E,
                                            int page_size, bool vec, bool pvec) {
  if (entry < g.NB) {
    if (pvec) {   // (a piece of four never crosses a page: rows and pages are multiples of four numbers)
      const size_t flat = (size_t)entry * width + col, per_page = (size_t)page_size * E;
      return load4(pooled + (size_t)g.table[flat / per_page] * per_page + flat % per_page);
    }
  } else if (vec) {
    const int p = g.j0 + entry - g.NB;
    return load4(cache + ((size_t)g.table[p / page_size] * page_size + p % page_size) * width + col);
  }
  float v[4];
#pragma unroll
  for (int y = 0; y < 4; ++y)
    v[y] = y < valid ? entry_value<T>(cache, pooled, g, entry, col + y, width, E, page_size) : 0.f;
  return make_float4(v[0], v[1], v[2], v[3]);
}

template <typename T>
__global__ __launch_bounds__(kSplitThreads) void pooled_values_kernel(const T* __restrict__ v_cache,
                                                                      T* __restrict__ out, SplitArgs a) {
  extern __shared__ float lds[];
  const int H = a.H, group = a.H / a.G, vdim = a.vdim, VW = a.G * a.vdim;
  const int c = blockIdx.y, split = blockIdx.z;
  float* wm = lds;                                   // [TQ * group][kSplitThreads] mixed weights of a chunk
  const int vdimp = (vdim + 3) & ~3, upr = vdimp / 4;   // a row padded to pieces of four channels
  float* Vs = wm + a.TQ * group * kSplitThreads;     // [kStage][vdimp] values of a stage
  const int tid = threadIdx.x;
  // thread (pg, cg): channels [4 cg, 4 cg + 4) of the pairs [pg PP, (pg + 1) PP)
  int CG = 1;
  while (CG < upr) CG *= 2;
  const int PG = kSplitThreads / CG, PP = (a.TQ * group + PG - 1) / PG;
  const int cg = tid & (CG - 1), pg = tid / CG;
  const bool owner = 4 * cg < vdim;
  const bool vvec = vdim % 4 == 0;
  const bool pvvec = vvec && ((long)a.page_size * a.VE) % 4 == 0;
  const int row_end = min(a.N, (int)(blockIdx.x + 1) * a.TQ);
  int row = blockIdx.x * a.TQ;
  while (row < row_end) {
    const Segment g = segment_at(a, row, row_end);
    const int pairs = g.tq * group;
    __syncthreads();
    const int e_lo = (int)((long)g.E * split / a.S), e_hi = (int)((long)g.E * (split + 1) / a.S);
    float acc[kOwnMax][4];
#pragma unroll
    for (int p = 0; p < kOwnMax; ++p)
#pragma unroll
      for (int d = 0; d < 4; ++d) acc[p][d] = 0.f;
    for (int e0 = e_lo; e0 < e_hi; e0 += kSplitThreads) {
      const int ne = min(kSplitThreads, e_hi - e0);
      __syncthreads();            // the chunk before is applied
      if (tid < ne) {
        for (int t = 0; t < g.tq; ++t) {
          const float* sc = a.scores + ((size_t)(g.row + t) * a.Emax + e0 + tid) * H + c * group;
          if (group % 4 == 0 && H % 4 == 0) {
#pragma unroll
            for (int h = 0; h < kGroupMax; h += 4) {
              if (h < group) {
                const float4 f = *reinterpret_cast<const float4*>(sc + h);
                wm[(t * group + h) * kSplitThreads + tid] = f.x;
                wm[(t * group + h + 1) * kSplitThreads + tid] = f.y;
                wm[(t * group + h + 2) * kSplitThreads + tid] = f.z;
                wm[(t * group + h + 3) * kSplitThreads + tid] = f.w;
              }
            }
          } else {
            for (int h = 0; h < group; ++h) wm[(t * group + h) * kSplitThreads + tid] = sc[h];
          }
        }
      }
      __syncthreads();
      // the chunk's values 64 entries at a time through LDS (every thread asks for four pieces of
      // four channels at once), then applied: a thread owns four channels of up to eight (row, head) pairs
      for (int sub = 0; sub < ne; sub += kStage) {
        const int nsub = min(kStage, ne - sub);
        const int units = nsub * upr;
        for (int i0 = tid; i0 < units; i0 += 4 * kSplitThreads) {
          float4 val[4];
#pragma unroll
          for (int y = 0; y < 4; ++y) {
            const int i = i0 + y * kSplitThreads;
            if (i < units) {
              const int e = i / upr, x = 4 * (i - e * upr);
              val[y] = load_unit<T>(v_cache, a.v_pool, g, e0 + sub + e, c * vdim + x, vdim - x, VW, a.VE, a.page_size,
                                    vvec, pvvec);
            }
          }
#pragma unroll
          for (int y = 0; y < 4; ++y) {
            const int i = i0 + y * kSplitThreads;
            if (i < units) {
              const int e = i / upr, x = 4 * (i - e * upr);
              *reinterpret_cast<float4*>(Vs + e * vdimp + x) = val[y];
            }
          }
        }
        __syncthreads();
        if (owner) {
          for (int e = 0; e < nsub; ++e) {
            const float4 v4 = *reinterpret_cast<const float4*>(Vs + e * vdimp + 4 * cg);
#pragma unroll
            for (int pp = 0; pp < kOwnMax; ++pp) {
              const int p = pg * PP + pp;
              if (pp < PP && p < pairs) {
                const float w = wm[p * kSplitThreads + sub + e];
                acc[pp][0] = fmaf(w, v4.x, acc[pp][0]);
                acc[pp][1] = fmaf(w, v4.y, acc[pp][1]);
                acc[pp][2] = fmaf(w, v4.z, acc[pp][2]);
                acc[pp][3] = fmaf(w, v4.w, acc[pp][3]);
              }
            }
          }
        }
        __syncthreads();        // before the next stage overwrites the values (and the next chunk the weights)
      }
    }
    if (owner) {
#pragma unroll
      for (int pp = 0; pp < kOwnMax; ++pp) {
        const int p = pg * PP + pp;
        if (pp < PP && p < pairs) {
          const int t = p / group, h = p % group;
#pragma unroll
          for (int y = 0; y < 4; ++y) {
            const int x = 4 * cg + y;
            if (x < vdim) {
              const size_t at = (size_t)(g.row + t) * H * vdim + (c * group + h) * vdim + x;
              if (a.S == 1) Elem<T>::store(out + at, acc[pp][y]);
              else a.part_o[(size_t)split * a.N * H * vdim + at] = acc[pp][y];
            }
          }
        }
      }
    }
    row += g.tq;
  }
}

template <typename T>
__global__ void pooled_merge_kernel(const float* __restrict__ part_o, T* __restrict__ out, int S, size_t total) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  float sum = 0.f;
  for (int s = 0; s < S; ++s) sum += part_o[(size_t)s * total + idx];
  Elem<T>::store(out + idx, sum);
}

// whether the score kernel's matrix-core form takes these operands (bfloat16 only)
template <typename T>
bool scores_on_matrix_cores(const void*, const void*, const SplitArgs&) { return false; }
template <>
bool scores_on_matrix_cores<bf16_t>(const void* q, const void* k_cache, const SplitArgs& a) {
  // (tiles of a portion's rows only: a single token's four or eight pairs fill an eighth of the 32 columns,
  // and its few entries a block are sooner walked a lane an entry: 34 against 41 us for 8 tokens over 2,058 positions)
  return a.TQ > 1 && a.dim % 16 == 0 && a.dim <= 16 * kStepsMax && ((uintptr_t)q % 16) == 0 &&
         ((uintptr_t)k_cache % 16) == 0;
}

template <typename T>
int launch_split(const void* q, const void* k_cache, const void* v_cache, void* out, const SplitArgs& a,
                 hipStream_t stream) {
  const int group = a.H / a.G;
  const dim3 grid((a.N + a.TQ - 1) / a.TQ, a.G, a.S);
  const size_t lds_a = ((size_t)a.TQ * group * a.dim + 2 * (kSplitThreads / kWave) * kPairMax * 2) * 4;
  const size_t work = (size_t)a.TQ * group * kSplitThreads + (size_t)kStage * ((a.vdim + 3) & ~3);
  const size_t lds_b = work * 4;
  const size_t lds_n = ((size_t)a.H * ((a.H + 3) & ~3) + 2 * a.H * a.S + 2 * a.H) * 4;
  if (lds_a > 150 * 1024 || lds_b > 150 * 1024 || lds_n > 64 * 1024) return -3;
  static bool allowed = false;      // (per instantiation: once per storage type)
  if (!allowed) {
    hipError_t err = hipFuncSetAttribute((const void*)pooled_scores_kernel<T>,
                                         hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (err == hipSuccess)
      err = hipFuncSetAttribute((const void*)pooled_values_kernel<T>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                160 * 1024);
    if (err != hipSuccess) return (int)err;
    allowed = true;
  }
  if (scores_on_matrix_cores<T>(q, k_cache, a)) {
    static bool mfma_allowed = false;
    if (!mfma_allowed) {
      const hipError_t err = hipFuncSetAttribute((const void*)pooled_scores_mfma_kernel,
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
      if (err != hipSuccess) return (int)err;
      mfma_allowed = true;
    }
    pooled_scores_mfma_kernel<<<grid, kSplitThreads, lds_a, stream>>>((const bf16_t*)q, (const bf16_t*)k_cache, a);
  } else {
    pooled_scores_kernel<T><<<grid, kSplitThreads, lds_a, stream>>>((const T*)q, (const T*)k_cache, a);
  }
  pooled_normalize_kernel<<<dim3(a.N, (a.Emax + kSplitThreads - 1) / kSplitThreads), kSplitThreads, lds_n, stream>>>(a);
  pooled_values_kernel<T><<<grid, kSplitThreads, lds_b, stream>>>((const T*)v_cache, (T*)out, a);
  if (a.S > 1) {
    const size_t total = (size_t)a.N * a.H * a.vdim;
    pooled_merge_kernel<T><<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(a.part_o, (T*)out, a.S, total);
  }
  return launch_status();
}

}  // namespace

// qkv: [N, QW + KW + VW] (QW alone if !store) in dtype, or float32 / float32 partial sums.
TK_API int tk_bias_norm_store(int dtype, const void* qkv, int in_f32, int parts, long part_stride,
                              const float* bias, const float* q_weight, const float* k_weight,
                              const int* positions, const int* req_of_token, const int* tables, int table_width,
                              void* q_out, void* k_cache, void* v_cache, int N, int QW, int KW, int VW,
                              int page_size, float eps, int store, hipStream_t stream) {
  if (N <= 0) return 0;
  if (QW < 1 || KW < 1 || VW < 1 || page_size < 1) return -2;
  const int total = store ? QW + KW + VW : QW;
  if (total <= kRowRegs * 1024) {
    const int threads = total >= 4096 ? 1024 : (total >= 1024 ? 512 : 256);
    if (dtype == 0)
      bias_norm_store_row_kernel<float><<<N, threads, 0, stream>>>(
          qkv, in_f32, parts, part_stride, bias, q_weight, k_weight, positions, req_of_token, tables, table_width,
          (float*)q_out, (float*)k_cache, (float*)v_cache, QW, KW, VW, page_size, eps, store);
    else
      bias_norm_store_row_kernel<bf16_t><<<N, threads, 0, stream>>>(
          qkv, in_f32, parts, part_stride, bias, q_weight, k_weight, positions, req_of_token, tables, table_width,
          (bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache, QW, KW, VW, page_size, eps, store);
    return launch_status();
  }
  if (dtype == 0)
    bias_norm_store_kernel<float><<<N, 256, 0, stream>>>(qkv, in_f32, parts, part_stride, bias, q_weight, k_weight,
                                                         positions, req_of_token, tables, table_width, (float*)q_out,
                                                         (float*)k_cache, (float*)v_cache, QW, KW, VW, page_size,
                                                         eps, store);
  else
    bias_norm_store_kernel<bf16_t><<<N, 256, 0, stream>>>(qkv, in_f32, parts, part_stride, bias, q_weight, k_weight,
                                                          positions, req_of_token, tables, table_width,
                                                          (bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache, QW, KW,
                                                          VW, page_size, eps, store);
  return launch_status();
}

// k_pool / v_pool: float32 paged arrays with KE / VE elements a position (>= ceil(width / pool))
TK_API int tk_pool_blocks(int dtype, const void* k_cache, const void* v_cache, float* k_pool, float* v_pool,
                          const int* positions, const int* req_of_token, const int* tables, int table_width, int N,
                          int KW, int VW, int KE, int VE, int pool, int page_size, hipStream_t stream) {
  if (N <= 0) return 0;
  if (pool < 1 || page_size < 1 || (long)KE * pool < KW || (long)VE * pool < VW) return -2;
  if (dtype == 0)
    pool_blocks_kernel<float><<<N, 256, 0, stream>>>((const float*)k_cache, (const float*)v_cache, k_pool, v_pool,
                                                     positions, req_of_token, tables, table_width, KW, VW, KE, VE,
                                                     pool, page_size);
  else
    pool_blocks_kernel<bf16_t><<<N, 256, 0, stream>>>((const bf16_t*)k_cache, (const bf16_t*)v_cache, k_pool, v_pool,
                                                      positions, req_of_token, tables, table_width, KW, VW, KE, VE,
                                                      pool, page_size);
  return launch_status();
}

// LDS bytes of a launch with tiles of TQ rows and chunks of CH entries
TK_API long tk_pooled_window_lds(int H, int G, int dim, int vdim, int TQ, int CH) {
  const long floats = (long)TQ * H * dim + (long)CH * (G * dim + 1) + (long)CH * (G * vdim + 1) +
                      2L * TQ * H * CH + 2L * TQ * H + (long)H * H;
  return floats * 4;
}

TK_API int tk_pooled_window_attention(int dtype, const void* q, const void* k_cache, const void* v_cache,
                                      const float* k_pool, const float* v_pool, int KE, int VE,
                                      void* out, const int* positions, const int* req_of_token,
                                      const int* q_start, const int* tables, int table_width, const float* talk,
                                      int N, int H, int G, int dim, int vdim, int size, int pool, int page_size,
                                      int TQ, int CH, int threads, float scale, hipStream_t stream) {
  if (N <= 0) return 0;
  if (H < 1 || G < 1 || H % G || dim < 1 || vdim < 1 || size < 1 || pool < 1 || page_size < 1 || TQ < 1 || CH < 1 ||
      threads % kWave || threads < kWave || threads > 1024 || (long)TQ * H * vdim > (long)kAcc * threads ||
      (long)KE * pool < (long)G * dim || (long)VE * pool < (long)G * vdim)
    return -2;
  const long lds = tk_pooled_window_lds(H, G, dim, vdim, TQ, CH);
  if (lds > 160 * 1024) return -3;
  PoolArgs a{positions, req_of_token, q_start, tables, talk, k_pool, v_pool, table_width, N, H, G, dim, vdim,
             size, pool, page_size, TQ, CH, KE, VE, scale};
  const unsigned blocks = (unsigned)((N + TQ - 1) / TQ);
  // the most LDS asked for so far is allowed once per kernel (not at every launch: a launch
  // may be recorded into a graph, whose first, eager run has then already raised the limit)
  static long allowed[2] = {0, 0};
  if (lds > allowed[dtype != 0]) {
    const void* fn = dtype == 0 ? (const void*)pooled_window_attention_kernel<float>
                                : (const void*)pooled_window_attention_kernel<bf16_t>;
    const hipError_t err = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (err != hipSuccess) return (int)err;
    allowed[dtype != 0] = 160 * 1024;
  }
  if (dtype == 0) {
    pooled_window_attention_kernel<float><<<blocks, threads, lds, stream>>>(
        (const float*)q, (const float*)k_cache, (const float*)v_cache, (float*)out, a);
  } else {
    pooled_window_attention_kernel<bf16_t><<<blocks, threads, lds, stream>>>(
        (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, (bf16_t*)out, a);
  }
  return launch_status();
}

// The four-kernel form.  scores [N, Emax, H], part_m / part_l [N, H, S], part_o [S, N, H * vdim]
// (unused if S == 1) are float32 scratch; Emax bounds the entries any tile of TQ rows sees.
TK_API int tk_pooled_window_attention_split(int dtype, const void* q, const void* k_cache, const void* v_cache,
                                            const float* k_pool, const float* v_pool, int KE, int VE, void* out,
                                            const int* positions, const int* req_of_token, const int* q_start,
                                            const int* tables, int table_width, const float* talk, float* scores,
                                            float* part_m, float* part_l, float* part_o, int N, int H, int G,
                                            int dim, int vdim, int size, int pool, int page_size, int TQ, int S,
                                            int Emax, float scale, hipStream_t stream) {
  if (N <= 0) return 0;
  if (H < 1 || H > kHeadsMax || G < 1 || H % G || H / G > kGroupMax || dim < 1 || vdim < 1 || vdim > 256 || size < 1 ||
      pool < 1 || page_size < 1 || TQ < 1 || TQ > kTileMax || TQ * (H / G) > kPairMax || S < 1 || Emax < 1 ||
      (long)KE * pool < (long)G * dim || (long)VE * pool < (long)G * vdim)
    return -2;
  SplitArgs a{positions, req_of_token, q_start, tables, talk, k_pool, v_pool, scores, part_m, part_l, part_o,
              table_width, N, H, G, dim, vdim, size, pool, page_size, TQ, S, Emax, KE, VE, scale};
  if (dtype == 0) return launch_split<float>(q, k_cache, v_cache, out, a, stream);
  return launch_split<bf16_t>(q, k_cache, v_cache, out, a, stream);
}

TK_SLOTS(tk_bias_norm_store)
TK_SLOTS(tk_pool_blocks)
TK_SLOTS(tk_pooled_window_attention)
TK_SLOTS(tk_pooled_window_attention_split)

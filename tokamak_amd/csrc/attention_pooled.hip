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

}  // namespace

// qkv: [N, QW + KW + VW] (QW alone if !store) in dtype, or float32 / float32 partial sums.
TK_API int tk_bias_norm_store(int dtype, const void* qkv, int in_f32, int parts, long part_stride,
                              const float* bias, const float* q_weight, const float* k_weight,
                              const int* positions, const int* req_of_token, const int* tables, int table_width,
                              void* q_out, void* k_cache, void* v_cache, int N, int QW, int KW, int VW,
                              int page_size, float eps, int store, hipStream_t stream) {
  if (N <= 0) return 0;
  if (QW < 1 || KW < 1 || VW < 1 || page_size < 1) return -2;
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

TK_SLOTS(tk_bias_norm_store)
TK_SLOTS(tk_pool_blocks)
TK_SLOTS(tk_pooled_window_attention)

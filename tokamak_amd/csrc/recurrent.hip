// Kernels of recurrent mixers with a matrix-valued state per head (gfx950).
//
// token_shift: per token the interpolations x + (x_prev - x) * mu_s between a row and the row
//   before it in its sequence; the row before a step's first token comes from the request's
//   state, which then takes the step's last row.
// tanh: the activation between the two products of a low-rank decay.
// wkv_scan: per (request, head) the recurrence
//     o_t = (S + diag(u) k_t v_t^T)^T r_t ;  S <- diag(w_t) S + k_t v_t^T ,  w_t = exp(-exp(d_t + w0))
//   over the step's tokens in order, the state S [dim, dim] in float32 registers (a thread owns a
//   few key channels of a column), followed by the head's unit norm, a gain and a SiLU gate.
//
// gla_scan: per (request, head) the gated linear attention recurrence
//     S <- diag(a_t) S + k_t v_t^T ;  o_t = S^T (q_t * q_scale) ,  a_t = sigmoid(z_t + b)^(1/tau)
//   with a state S [dim, vdim] whose two sides may differ, the newest token already in S when it
//   is read, followed by the head's unit norm, a gain per value channel and a SiLU gate.
//
// Decays, exponentials, the state and the norm are float32 whatever the storage type.
#include "common.h"
#include "slots.h"

using namespace tk;

namespace {

// element idx of a [rows, width] input: T, or float32, or the sum of float32 partial sums
template <typename T>
__device__ __forceinline__ float load_in(const void* p, int f32, int parts, long part_stride, size_t idx) {
  if (!f32) return Elem<T>::load(reinterpret_cast<const T*>(p) + idx);
  const float* f = reinterpret_cast<const float*>(p) + idx;
  float s = f[0];
  int i = 1;
  for (; i + 3 < parts; i += 4) {      // four loads in flight; the sums in the order of the parts
    const float a = f[(size_t)i * part_stride], b = f[(size_t)(i + 1) * part_stride];
    const float c = f[(size_t)(i + 2) * part_stride], d = f[(size_t)(i + 3) * part_stride];
    s = (((s + a) + b) + c) + d;
  }
  for (; i < parts; ++i) s += f[(size_t)i * part_stride];
  return s;
}

// VEC consecutive elements of T as one 16-byte access (VEC = 4 float32 or 8 bfloat16)
template <typename T, int VEC> __device__ __forceinline__ void load_vec(const T* p, float* o);
template <> __device__ __forceinline__ void load_vec<float, 4>(const float* p, float* o) {
  const float4 v = *reinterpret_cast<const float4*>(p);
  o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
}
template <> __device__ __forceinline__ void load_vec<bf16_t, 8>(const bf16_t* p, float* o) {
  const uint4 v = *reinterpret_cast<const uint4*>(p);
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    o[2 * i] = __uint_as_float(w[i] << 16);
    o[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}
template <typename T, int VEC> __device__ __forceinline__ void store_vec(T* p, const float* o);
template <> __device__ __forceinline__ void store_vec<float, 4>(float* p, const float* o) {
  *reinterpret_cast<float4*>(p) = make_float4(o[0], o[1], o[2], o[3]);
}
template <> __device__ __forceinline__ void store_vec<bf16_t, 8>(bf16_t* p, const float* o) {
  *reinterpret_cast<uint4*>(p) = make_uint4(pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3]), pack_bf16x2(o[4], o[5]),
                                            pack_bf16x2(o[6], o[7]));
}

template <typename T>
__global__ void token_shift_kernel(const T* __restrict__ h, const float* __restrict__ mu,
                                   float* __restrict__ last, T* __restrict__ out,
                                   const int* __restrict__ req_of_token, const int* __restrict__ q_start,
                                   const int* __restrict__ state_slots, int N, int W, int S) {
  const int n = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;      // a thread a column: no loop whose loads wait for one another
  if (c >= W) return;
  const int r = req_of_token[n];
  const int first = q_start[r];
  const int end = q_start[r + 1];
  const bool head = n == first;
  float* mine = last + (size_t)state_slots[r] * W;
  const float cur = Elem<T>::load(h + (size_t)n * W + c);
  const float prev = head ? mine[c] : Elem<T>::load(h + (size_t)(n - 1) * W + c);
  const float newest = head ? Elem<T>::load(h + (size_t)(end - 1) * W + c) : 0.f;
  const float d = prev - cur;
  for (int s = 0; s < S; ++s)
    Elem<T>::store(out + ((size_t)s * N + n) * W + c, cur + d * mu[(size_t)s * W + c]);
  // the thread that has read the old row of the state is the one that replaces it
  if (head) mine[c] = newest;
}

// The same, a thread VEC consecutive columns (16 bytes of a row of T): W a multiple of VEC.
template <typename T, int VEC>
__global__ void token_shift_vec_kernel(const T* __restrict__ h, const float* __restrict__ mu,
                                       float* __restrict__ last, T* __restrict__ out,
                                       const int* __restrict__ req_of_token, const int* __restrict__ q_start,
                                       const int* __restrict__ state_slots, int N, int W, int S) {
  const int n = blockIdx.x;
  const int c = (blockIdx.y * blockDim.x + threadIdx.x) * VEC;
  if (c >= W) return;
  const int r = req_of_token[n];
  const int first = q_start[r];
  const int end = q_start[r + 1];
  const bool head = n == first;
  float* mine = last + (size_t)state_slots[r] * W;
  float cur[VEC], prev[VEC], newest[VEC];
  load_vec<T, VEC>(h + (size_t)n * W + c, cur);
  if (head) {
#pragma unroll
    for (int y = 0; y < VEC; y += 4) {
      const float4 v = *reinterpret_cast<const float4*>(mine + c + y);
      prev[y] = v.x; prev[y + 1] = v.y; prev[y + 2] = v.z; prev[y + 3] = v.w;
    }
    load_vec<T, VEC>(h + (size_t)(end - 1) * W + c, newest);
  } else {
    load_vec<T, VEC>(h + (size_t)(n - 1) * W + c, prev);
  }
  for (int s = 0; s < S; ++s) {
    float o[VEC];
#pragma unroll
    for (int y = 0; y < VEC; y += 4) {
      const float4 m = *reinterpret_cast<const float4*>(mu + (size_t)s * W + c + y);
      o[y] = cur[y] + (prev[y] - cur[y]) * m.x;
      o[y + 1] = cur[y + 1] + (prev[y + 1] - cur[y + 1]) * m.y;
      o[y + 2] = cur[y + 2] + (prev[y + 2] - cur[y + 2]) * m.z;
      o[y + 3] = cur[y + 3] + (prev[y + 3] - cur[y + 3]) * m.w;
    }
    store_vec<T, VEC>(out + ((size_t)s * N + n) * W + c, o);
  }
  if (head) {
#pragma unroll
    for (int y = 0; y < VEC; y += 4)
      *reinterpret_cast<float4*>(mine + c + y) = make_float4(newest[y], newest[y + 1], newest[y + 2], newest[y + 3]);
  }
}

template <typename T>
__global__ void tanh_kernel(const void* __restrict__ in, int f32, int parts, long part_stride,
                            T* __restrict__ out, size_t total) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  Elem<T>::store(out + idx, tanhf(load_in<T>(in, f32, parts, part_stride, idx)));
}

constexpr int kScanTokens = 8;   // tokens whose operands are staged in LDS at once

// an operand [N, heads * dim]: T, or float32, or float32 partial sums of a split product
struct ScanIn {
  const void* p;
  int f32, parts;
  long stride;
};

// PLAIN: the operand is known to be T (a long portion's products): one load, no branch
template <typename T, bool PLAIN>
__device__ __forceinline__ float scan_load(const ScanIn& in, size_t idx) {
  if (PLAIN) return Elem<T>::load(reinterpret_cast<const T*>(in.p) + idx);
  return load_in<T>(in.p, in.f32, in.parts, in.stride, idx);
}

struct ScanShape {
  int heads, dim, columns, slices, slice;   // threads = columns * slices; a thread owns `slice` key channels of a column
};

// A block a (request, head).  Thread (ks, j) owns the state's rows [ks * slice, (ks + 1) * slice)
// of column j in registers: the key channels of a head are cut over `slices` groups of threads, so
// that a token costs each thread `slice` multiply-adds and not `dim`; the groups' partial
// outputs meet in LDS.  Tokens run in order, eight staged at a time.
template <typename T, int SLICE, bool PLAIN>
__global__ __launch_bounds__(1024) void wkv_scan_kernel(
    ScanIn r_in, ScanIn k_in, ScanIn v_in, ScanIn g_in, ScanIn d_in,
    const float* __restrict__ w0, const float* __restrict__ u, const float* __restrict__ gain,
    float* __restrict__ state, const int* __restrict__ q_start, const int* __restrict__ state_slots,
    T* __restrict__ out, ScanShape sh, float eps) {
  constexpr int TB = kScanTokens;
  extern __shared__ float lds[];
  const int dim = sh.dim, CT = sh.columns, KS = sh.slices, slice = sh.slice;
  const int dimp = (dim + 3) & ~3;
  float* rr = lds;                     // [TB][dimp] each
  float* kk = rr + TB * dimp;
  float* ww = kk + TB * dimp;
  float* uk = ww + TB * dimp;
  float* os = uk + TB * dimp;
  float* rstd = os + TB * dimp;        // [TB]
  float* part = rstd + TB;             // [KS][TB][CT]
  const int req = blockIdx.x, head = blockIdx.y;
  const int tid = threadIdx.x, nthreads = blockDim.x;
  const int ks = tid / CT, j = tid - ks * CT;
  const bool live = j < dim;
  const int k0 = ks * slice;
  const int kn = max(0, min(slice, dim - k0));     // key channels of this thread's slice that exist
  const int HD = sh.heads * dim;
  const int base = head * dim;
  const int first = q_start[req], end = q_start[req + 1];
  float* S = state + ((size_t)state_slots[req] * sh.heads + head) * dim * dim;
  float s[SLICE];
#pragma unroll
  for (int x = 0; x < SLICE; ++x) s[x] = (live && x < kn) ? S[(size_t)(k0 + x) * dim + j] : 0.f;
  const float gj = live ? gain[base + j] : 0.f;
  const int lane = tid & (kWave - 1), wave = tid / kWave, nwaves = nthreads / kWave;

  for (int t0 = first; t0 < end; t0 += TB) {
    const int tb = min(TB, end - t0);
    for (int i = tid; i < tb * dim; i += nthreads) {
      const int t = i / dim, c = i - t * dim;
      const size_t at = (size_t)(t0 + t) * HD + base + c;
      const float kv = scan_load<T, PLAIN>(k_in, at);
      rr[t * dimp + c] = scan_load<T, PLAIN>(r_in, at);
      kk[t * dimp + c] = kv;
      uk[t * dimp + c] = u[base + c] * kv;
      ww[t * dimp + c] = expf(-expf(scan_load<T, false>(d_in, at) + w0[base + c]));
    }
    float vloc[TB];
#pragma unroll
    for (int t = 0; t < TB; ++t)
      vloc[t] = (t < tb && live) ? scan_load<T, PLAIN>(v_in, (size_t)(t0 + t) * HD + base + j) : 0.f;
    __syncthreads();
#pragma unroll
    for (int t = 0; t < TB; ++t) {
      if (t < tb) {
        const float vj = vloc[t];
        float o = 0.f;
#pragma unroll
        for (int x = 0; x < SLICE; x += 4) {
          if (x < kn) {
            const int at = t * dimp + k0 + x;       // (k0 and dimp are multiples of four)
            const float4 r4 = *reinterpret_cast<const float4*>(rr + at);
            const float4 k4 = *reinterpret_cast<const float4*>(kk + at);
            const float4 w4 = *reinterpret_cast<const float4*>(ww + at);
            const float4 u4 = *reinterpret_cast<const float4*>(uk + at);
            const float rv[4] = {r4.x, r4.y, r4.z, r4.w}, kv[4] = {k4.x, k4.y, k4.z, k4.w};
            const float wv[4] = {w4.x, w4.y, w4.z, w4.w}, uv[4] = {u4.x, u4.y, u4.z, u4.w};
#pragma unroll
            for (int y = 0; y < 4; ++y) {
              if (x + y < kn) {
                o = fmaf(rv[y], fmaf(uv[y], vj, s[x + y]), o);
                s[x + y] = fmaf(wv[y], s[x + y], kv[y] * vj);
              }
            }
          }
        }
        part[(ks * TB + t) * CT + j] = o;
      }
    }
    __syncthreads();
    for (int t = ks; t < tb; t += KS) {
      float o = 0.f;
      for (int q = 0; q < KS; ++q) o += part[(q * TB + t) * CT + j];
      if (live) os[t * dimp + j] = o;
    }
    __syncthreads();
    for (int t = wave; t < tb; t += nwaves) {
      float q = 0.f;
      for (int x = lane; x < dim; x += kWave) q += os[t * dimp + x] * os[t * dimp + x];
      q = wave_sum(q);
      if (lane == 0) rstd[t] = 1.f / sqrtf(q / (float)dim + eps);
    }
    __syncthreads();
    for (int t = ks; t < tb; t += KS) {
      if (live) {
        const size_t at = (size_t)(t0 + t) * HD + base + j;
        const float g = scan_load<T, PLAIN>(g_in, at);
        Elem<T>::store(out + at, os[t * dimp + j] * rstd[t] * gj * (g / (1.f + expf(-g))));
      }
    }
    // (the next round's staging writes rr, kk, ww, uk, which nobody reads after the second
    // barrier; os, rstd and part are written again only behind the next round's barriers)
  }
  if (live) {
#pragma unroll
    for (int x = 0; x < SLICE; ++x)
      if (x < kn) S[(size_t)(k0 + x) * dim + j] = s[x];
  }
}

template <typename T>
int launch_scan(ScanIn r, ScanIn k, ScanIn v, ScanIn g, ScanIn d, const float* w0, const float* u, const float* gain, float* state,
                const int* q_start, const int* state_slots, void* out, int R, int heads, int dim, float eps,
                hipStream_t stream) {
  ScanShape sh;
  sh.heads = heads;
  sh.dim = dim;
  sh.columns = (dim + kWave - 1) / kWave * kWave;
  const int most = min(16, 1024 / sh.columns);                      // groups of threads that can share a head
  sh.slice = max(4, ((dim + most - 1) / most + 3) / 4 * 4);
  sh.slices = (dim + sh.slice - 1) / sh.slice;
  const int threads = sh.columns * sh.slices;
  const int dimp = (dim + 3) & ~3;
  const size_t lds = ((size_t)5 * kScanTokens * dimp + kScanTokens + (size_t)sh.slices * kScanTokens * sh.columns) * 4;
  const dim3 grid(R, heads);
  const bool plain = !r.f32 && !k.f32 && !v.f32 && !g.f32;
#define TK_SCAN_AS(SLICE, PLAIN)                                                                              \
  {                                                                                                           \
    static bool allowed = false;                                                                              \
    if (!allowed) {                                                                                           \
      const hipError_t err = hipFuncSetAttribute((const void*)wkv_scan_kernel<T, SLICE, PLAIN>,               \
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);     \
      if (err != hipSuccess) return (int)err;                                                                 \
      allowed = true;                                                                                         \
    }                                                                                                         \
    wkv_scan_kernel<T, SLICE, PLAIN><<<grid, threads, lds, stream>>>(r, k, v, g, d, w0, u, gain, state,       \
                                                                     q_start, state_slots, (T*)out, sh, eps); \
  }
#define TK_SCAN(SLICE)                 \
  {                                    \
    if (plain) TK_SCAN_AS(SLICE, true) \
    else TK_SCAN_AS(SLICE, false)      \
  }
  if (sh.slice <= 4) TK_SCAN(4)
  else if (sh.slice <= 16) TK_SCAN(16)
  else TK_SCAN(64)
#undef TK_SCAN_AS
#undef TK_SCAN
  return launch_status();
}

struct GlaShape {
  int heads, dim, vdim, columns, slices, slice;   // threads = columns * slices; a thread owns `slice` key channels of a value column
  int splits;                                     // blocks that share a head's value columns (blockIdx.z), `columns` each
};

// A block a (request, head, share of the value columns).  Thread (ks, j) owns rows
// [ks * slice, (ks + 1) * slice) of one column (a value channel) of the state in registers; the
// groups' partial outputs meet in LDS.  Tokens run in order, eight staged at a time.
// a = sigmoid(z)^(1/tau) is formed as exp(-softplus(-z) / tau), softplus(x) = max(x, 0) + log1p(exp(-|x|)).
// The columns of the state never meet (column j of S only ever sees v[j]), so a head's columns may
// be cut over several blocks: a long portion of one request then fills more of the GPU, and a
// block's waves, which all read every token's q, k and a from LDS, are fewer.  Only the head's norm
// needs all columns: with several shares the kernel leaves the raw o in `raw` (float32) and
// gla_finish_kernel applies norm, gain and gate; the decays, which every share would form again
// from z, are then made once by gla_decay_kernel (READY: z_in holds them, float32).
// Measured on a 2,048-token portion of 32 heads of 128 x 128: one block a head 2.85 ms; eight
// shares of 16 columns 2.43 ms; rounds of 32 tokens instead of 8 no faster (3.0 ms: a round's time
// is its tokens' dependent steps, not its barriers); a round's operands asked for a round ahead and
// kept in registers meanwhile 3.1 ms against 2.3.
template <typename T, int SLICE, bool PLAIN, bool READY>
__global__ __launch_bounds__(1024) void gla_scan_kernel(
    ScanIn q_in, ScanIn k_in, ScanIn v_in, ScanIn g_in, ScanIn z_in, const float* __restrict__ bias,
    const float* __restrict__ gain, float* __restrict__ state, const int* __restrict__ q_start,
    const int* __restrict__ state_slots, T* __restrict__ out, float* __restrict__ raw, GlaShape sh, float q_scale,
    float inv_tau, float eps) {
  constexpr int TB = kScanTokens;
  extern __shared__ float lds[];
  const int dim = sh.dim, vdim = sh.vdim, CT = sh.columns, KS = sh.slices, slice = sh.slice;
  const int dimp = (dim + 3) & ~3, vdimp = (vdim + 3) & ~3;
  float* qq = lds;                     // [TB][dimp] each
  float* kk = qq + TB * dimp;
  float* aa = kk + TB * dimp;
  float* os = aa + TB * dimp;          // [TB][vdimp]
  float* rstd = os + TB * vdimp;       // [TB]
  float* part = rstd + TB;             // [KS][TB][CT]
  const int req = blockIdx.x, head = blockIdx.y;
  const int tid = threadIdx.x, nthreads = blockDim.x;
  const int ks = tid / CT, jl = tid - ks * CT;
  const int j = blockIdx.z * CT + jl;               // the thread's value column; jl: its place in the block
  const bool worker = ks < KS;                      // (threads that only fill the last wave own nothing)
  const bool live = worker && j < vdim && jl < CT;
  const int k0 = ks * slice;
  const int kn = max(0, min(slice, dim - k0));     // key channels of this thread's slice that exist
  const int KW = sh.heads * dim, VW = sh.heads * vdim;
  const int kbase = head * dim, vbase = head * vdim;
  const int first = q_start[req], end = q_start[req + 1];
  float* S = state + ((size_t)state_slots[req] * sh.heads + head) * dim * vdim;
  float s[SLICE];
#pragma unroll
  for (int x = 0; x < SLICE; ++x) s[x] = (live && x < kn) ? S[(size_t)(k0 + x) * vdim + j] : 0.f;
  const float gj = live ? gain[j] : 0.f;
  const int lane = tid & (kWave - 1), wave = tid / kWave, nwaves = nthreads / kWave;

  for (int t0 = first; t0 < end; t0 += TB) {
    const int tb = min(TB, end - t0);
    for (int i = tid; i < tb * dim; i += nthreads) {
      const int t = i / dim, c = i - t * dim;
      const size_t at = (size_t)(t0 + t) * KW + kbase + c;
      qq[t * dimp + c] = scan_load<T, PLAIN>(q_in, at) * q_scale;
      kk[t * dimp + c] = scan_load<T, PLAIN>(k_in, at);
      if (READY) {
        aa[t * dimp + c] = reinterpret_cast<const float*>(z_in.p)[at];     // (the decay itself, made by gla_decay_kernel)
      } else {
        const float x = -(scan_load<T, false>(z_in, at) + bias[kbase + c]);
        aa[t * dimp + c] = expf(-(fmaxf(x, 0.f) + log1pf(expf(-fabsf(x)))) * inv_tau);
      }
    }
    float vloc[TB];
#pragma unroll
    for (int t = 0; t < TB; ++t)
      vloc[t] = (t < tb && live) ? scan_load<T, PLAIN>(v_in, (size_t)(t0 + t) * VW + vbase + j) : 0.f;
    __syncthreads();
#pragma unroll
    for (int t = 0; t < TB; ++t) {
      if (t < tb) {
        const float vj = vloc[t];
        float o = 0.f;
#pragma unroll
        for (int x = 0; x < SLICE; x += 4) {
          if (x < kn) {
            const int at = t * dimp + k0 + x;       // (k0 and dimp are multiples of four)
            const float4 q4 = *reinterpret_cast<const float4*>(qq + at);
            const float4 k4 = *reinterpret_cast<const float4*>(kk + at);
            const float4 a4 = *reinterpret_cast<const float4*>(aa + at);
            const float qv[4] = {q4.x, q4.y, q4.z, q4.w}, kv[4] = {k4.x, k4.y, k4.z, k4.w};
            const float av[4] = {a4.x, a4.y, a4.z, a4.w};
#pragma unroll
            for (int y = 0; y < 4; ++y) {
              if (x + y < kn) {
                s[x + y] = fmaf(av[y], s[x + y], kv[y] * vj);
                o = fmaf(qv[y], s[x + y], o);
              }
            }
          }
        }
        if (worker) part[(ks * TB + t) * CT + jl] = o;
      }
    }
    __syncthreads();
    for (int t = worker ? ks : tb; t < tb; t += KS) {
      float o = 0.f;
      for (int q = 0; q < KS; ++q) o += part[(q * TB + t) * CT + jl];
      if (live) {
        if (raw != nullptr) raw[(size_t)(t0 + t) * VW + vbase + j] = o;
        else os[t * vdimp + j] = o;
      }
    }
    __syncthreads();
    if (raw != nullptr) continue;      // (every thread of the block alike; the next round's staging is behind this barrier)
    for (int t = wave; t < tb; t += nwaves) {
      float q = 0.f;
      for (int x = lane; x < vdim; x += kWave) q += os[t * vdimp + x] * os[t * vdimp + x];
      q = wave_sum(q);
      if (lane == 0) rstd[t] = 1.f / sqrtf(q / (float)vdim + eps);
    }
    __syncthreads();
    for (int t = worker ? ks : tb; t < tb; t += KS) {
      if (live) {
        const size_t at = (size_t)(t0 + t) * VW + vbase + j;
        const float g = scan_load<T, PLAIN>(g_in, at);
        Elem<T>::store(out + at, os[t * vdimp + j] * rstd[t] * gj * (g / (1.f + expf(-g))));
      }
    }
    // (the next round's staging writes qq, kk, aa, which nobody reads after the second barrier;
    // os, rstd and part are written again only behind the next round's barriers)
  }
  if (live) {
#pragma unroll
    for (int x = 0; x < SLICE; ++x)
      if (x < kn) S[(size_t)(k0 + x) * vdim + j] = s[x];
  }
}

// a = sigmoid(z + b)^(1 / tau) for every (token, key channel), float32
template <typename T>
__global__ void gla_decay_kernel(ScanIn z_in, const float* __restrict__ bias, float* __restrict__ decay, int KW,
                                 float inv_tau, size_t total) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const float x = -(load_in<T>(z_in.p, z_in.f32, z_in.parts, z_in.stride, idx) + bias[idx % KW]);
  decay[idx] = expf(-(fmaxf(x, 0.f) + log1pf(expf(-fabsf(x)))) * inv_tau);
}

// out = o / rms(o) * gain * silu(gate) per (token, head), from the raw o that a scan with shared
// columns left: a wave a (token, head).
template <typename T>
__global__ __launch_bounds__(256) void gla_finish_kernel(const float* __restrict__ raw, ScanIn g_in,
                                                         const float* __restrict__ gain, T* __restrict__ out,
                                                         int pairs, int heads, int vdim, float eps) {
  const int lane = threadIdx.x & (kWave - 1);
  const int pair = blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (pair >= pairs) return;
  const size_t at = (size_t)pair * vdim;       // (token * heads + head) * vdim
  float q = 0.f;
  for (int x = lane; x < vdim; x += kWave) q += raw[at + x] * raw[at + x];
  q = wave_sum(q);
  const float rstd = 1.f / sqrtf(q / (float)vdim + eps);
  for (int x = lane; x < vdim; x += kWave) {
    const float g = load_in<T>(g_in.p, g_in.f32, g_in.parts, g_in.stride, at + x);
    Elem<T>::store(out + at + x, raw[at + x] * rstd * gain[x] * (g / (1.f + expf(-g))));
  }
}

template <typename T>
int launch_gla(ScanIn q, ScanIn k, ScanIn v, ScanIn g, ScanIn z, const float* bias, const float* gain, float* state,
               const int* q_start, const int* state_slots, void* out, float* raw, int N, int splits, int R, int heads,
               int dim, int vdim, float q_scale, float inv_tau, float eps, hipStream_t stream) {
  GlaShape sh;
  sh.heads = heads;
  sh.dim = dim;
  sh.vdim = vdim;
  sh.splits = splits;
  // a block's columns: the whole head in whole waves, or a share of 16 or more
  sh.columns = splits > 1 ? (vdim + splits - 1) / splits : (vdim + kWave - 1) / kWave * kWave;
  const int most = min(16, 1024 / sh.columns);                      // groups of threads that can share a head
  sh.slice = max(4, ((dim + most - 1) / most + 3) / 4 * 4);
  sh.slices = (dim + sh.slice - 1) / sh.slice;
  const int threads = (sh.columns * sh.slices + kWave - 1) / kWave * kWave;
  const int dimp = (dim + 3) & ~3, vdimp = (vdim + 3) & ~3;
  const size_t lds = ((size_t)3 * kScanTokens * dimp + (size_t)kScanTokens * vdimp + kScanTokens +
                      (size_t)sh.slices * kScanTokens * sh.columns) * 4;
  const bool ready = splits > 1;
  if (ready) {
    // the decays once for all shares, behind the raw outputs in the same scratch array
    float* decay = raw + (size_t)N * heads * vdim;
    const size_t total = (size_t)N * heads * dim;
    gla_decay_kernel<T><<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(z, bias, decay, heads * dim, inv_tau, total);
    z = ScanIn{decay, 1, 1, 0};
  }
  const dim3 grid(R, heads, splits);
  float* raw_out = splits > 1 ? raw : nullptr;
  const bool plain = !q.f32 && !k.f32 && !v.f32 && !g.f32;
#define TK_GLA_AS(SLICE, PLAIN, READY_)                                                                       \
  {                                                                                                           \
    static bool allowed = false;                                                                              \
    if (!allowed) {                                                                                           \
      const hipError_t err = hipFuncSetAttribute((const void*)gla_scan_kernel<T, SLICE, PLAIN, READY_>,       \
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);     \
      if (err != hipSuccess) return (int)err;                                                                 \
      allowed = true;                                                                                         \
    }                                                                                                         \
    gla_scan_kernel<T, SLICE, PLAIN, READY_><<<grid, threads, lds, stream>>>(q, k, v, g, z, bias, gain, state, \
                                                                             q_start, state_slots, (T*)out,   \
                                                                             raw_out, sh, q_scale, inv_tau, eps); \
  }
#define TK_GLA(SLICE)                                                   \
  {                                                                     \
    if (ready) {                                                        \
      if (plain) TK_GLA_AS(SLICE, true, true)                           \
      else TK_GLA_AS(SLICE, false, true)                                \
    } else if (plain) TK_GLA_AS(SLICE, true, false)                     \
    else TK_GLA_AS(SLICE, false, false)                                 \
  }
  if (sh.slice <= 4) TK_GLA(4)
  else if (sh.slice <= 16) TK_GLA(16)
  else TK_GLA(64)
#undef TK_GLA_AS
#undef TK_GLA
  if (splits > 1) {
    const int pairs = N * heads;
    gla_finish_kernel<T><<<(pairs + 3) / 4, 256, 0, stream>>>(raw, g, gain, (T*)out, pairs, heads, vdim, eps);
  }
  return launch_status();
}

}  // namespace

// out[s][n] = h[n] + (prev(n) - h[n]) * mu[s]; `last` [slots, W] float32 holds each request's
// newest row.  h, out: dtype (0 float32, 1 bfloat16).
TK_API int tk_token_shift(int dtype, const void* h, const float* mu, float* last, void* out,
                          const int* req_of_token, const int* q_start, const int* state_slots, int N, int W,
                          int S, hipStream_t stream) {
  if (N <= 0 || W <= 0 || S <= 0) return 0;
  const int vec = dtype == 0 ? 4 : 8;
  if (W % vec == 0) {      // (rows, the state's rows and the mix weights then all start on 16-byte borders)
    const int columns = W / vec;
    const int threads = columns >= 256 ? 256 : 64;
    const dim3 grid(N, (columns + threads - 1) / threads);
    if (dtype == 0)
      token_shift_vec_kernel<float, 4><<<grid, threads, 0, stream>>>((const float*)h, mu, last, (float*)out,
                                                                     req_of_token, q_start, state_slots, N, W, S);
    else
      token_shift_vec_kernel<bf16_t, 8><<<grid, threads, 0, stream>>>((const bf16_t*)h, mu, last, (bf16_t*)out,
                                                                      req_of_token, q_start, state_slots, N, W, S);
    return launch_status();
  }
  const int threads = W >= 256 ? 256 : 64;
  const dim3 grid(N, (W + threads - 1) / threads);
  if (dtype == 0)
    token_shift_kernel<float><<<grid, threads, 0, stream>>>((const float*)h, mu, last, (float*)out, req_of_token,
                                                         q_start, state_slots, N, W, S);
  else
    token_shift_kernel<bf16_t><<<grid, threads, 0, stream>>>((const bf16_t*)h, mu, last, (bf16_t*)out, req_of_token,
                                                          q_start, state_slots, N, W, S);
  return launch_status();
}

TK_API int tk_tanh(int dtype, const void* in, int in_f32, int parts, long part_stride, void* out, long total,
                   hipStream_t stream) {
  if (total <= 0) return 0;
  const unsigned blocks = (unsigned)((total + 255) / 256);
  if (dtype == 0)
    tanh_kernel<float><<<blocks, 256, 0, stream>>>(in, in_f32, parts, part_stride, (float*)out, (size_t)total);
  else
    tanh_kernel<bf16_t><<<blocks, 256, 0, stream>>>(in, in_f32, parts, part_stride, (bf16_t*)out, (size_t)total);
  return launch_status();
}

// r, k, v, g (gate), d (the decay's pre-activation): [N, heads * dim] in dtype, or float32, or
// float32 partial sums [parts, N, heads * dim]; out in dtype; state [slots, heads, dim, dim]
// float32.  dim <= 256.
TK_API int tk_wkv_scan(int dtype, const void* r, int r_f32, int r_parts, long r_stride, const void* k, int k_f32,
                       int k_parts, long k_stride, const void* v, int v_f32, int v_parts, long v_stride,
                       const void* g, int g_f32, int g_parts, long g_stride, const void* d, int d_f32, int d_parts,
                       long d_stride, const float* w0, const float* u, const float* gain, float* state,
                       const int* q_start, const int* state_slots, void* out, int R, int heads, int dim, float eps,
                       hipStream_t stream) {
  if (R <= 0 || heads <= 0) return 0;
  if (dim < 1 || dim > 256) return -2;
  const ScanIn ri{r, r_f32, r_parts, r_stride}, ki{k, k_f32, k_parts, k_stride}, vi{v, v_f32, v_parts, v_stride},
      gi{g, g_f32, g_parts, g_stride}, di{d, d_f32, d_parts, d_stride};
  if (dtype == 0)
    return launch_scan<float>(ri, ki, vi, gi, di, w0, u, gain, state, q_start, state_slots, out, R, heads, dim, eps,
                              stream);
  return launch_scan<bf16_t>(ri, ki, vi, gi, di, w0, u, gain, state, q_start, state_slots, out, R, heads, dim, eps,
                             stream);
}

// q, k, z (the decay's pre-activation, to which `bias` is added): [N, heads * dim]; v, g (gate):
// [N, heads * vdim]; each in dtype, or float32, or float32 partial sums [parts, N, width]; out
// [N, heads * vdim] in dtype; state [slots, heads, dim, vdim] float32.  dim, vdim <= 256.
// splits > 1: so many blocks share a head's value columns (8 or more each) and leave the raw o in
// raw (float32 [N, heads * vdim], and behind it room for the decays, [N, heads * dim]), which a
// second kernel norms and gates.
TK_API int tk_gla_scan(int dtype, const void* q, int q_f32, int q_parts, long q_stride, const void* k, int k_f32,
                       int k_parts, long k_stride, const void* v, int v_f32, int v_parts, long v_stride,
                       const void* g, int g_f32, int g_parts, long g_stride, const void* z, int z_f32, int z_parts,
                       long z_stride, const float* bias, const float* gain, float* state, const int* q_start,
                       const int* state_slots, void* out, float* raw, int N, int splits, int R, int heads, int dim,
                       int vdim, float q_scale, float inv_tau, float eps, hipStream_t stream) {
  if (R <= 0 || heads <= 0) return 0;
  if (dim < 1 || dim > 256 || vdim < 1 || vdim > 256) return -2;
  // shares of a head's columns: 8 columns or more each, and then the raw outputs need a place
  if (splits < 1 || (splits > 1 && (raw == nullptr || (vdim + splits - 1) / splits < 8))) return -1;
  const ScanIn qi{q, q_f32, q_parts, q_stride}, ki{k, k_f32, k_parts, k_stride}, vi{v, v_f32, v_parts, v_stride},
      gi{g, g_f32, g_parts, g_stride}, zi{z, z_f32, z_parts, z_stride};
  if (dtype == 0)
    return launch_gla<float>(qi, ki, vi, gi, zi, bias, gain, state, q_start, state_slots, out, raw, N, splits, R, heads,
                             dim, vdim, q_scale, inv_tau, eps, stream);
  return launch_gla<bf16_t>(qi, ki, vi, gi, zi, bias, gain, state, q_start, state_slots, out, raw, N, splits, R, heads,
                            dim, vdim, q_scale, inv_tau, eps, stream);
}

TK_SLOTS(tk_token_shift)
TK_SLOTS(tk_tanh)
TK_SLOTS(tk_wkv_scan)
TK_SLOTS(tk_gla_scan)

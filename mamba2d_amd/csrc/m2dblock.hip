// m2dblock.hip -- memory-bound operators of an M2D residual block that the stock libraries serve
// badly on gfx950 at this model's shapes, or in several passes where one will do: LayerNorm over
// a short channel axis (64 to 512 channels: models/mamba2d.py:57,220,248,363, models/utils.py:13,
// 232-233), the depthwise 3x3 convolution of the local path on channel-last tensors
// (models/utils.py:101-114), StarReLU (models/utils.py:26-44), the scaled residual sum
// (models/mamba2d.py:258-259), the rotary embedding + LayerNorm of q and k in the attention stages,
// and that attention as a whole where a head is 32 wide and the grid has up to 256 cells.  Inference
// forward only; each reads every input byte once and writes every output byte once.
//
// Layout: activations are row-major (rows, C) / (B, H, W, C), element type float or bf16; weights
// are float or bf16, independently of the activations (a bf16 model holds bf16 weights, a fp32
// model under autocast hands fp32 weights to bf16 activations).  Arithmetic is fp32.
#include <hip/hip_runtime.h>

#include <atomic>
#include <stdint.h>

#include "../../include/m2dscan.h"

namespace {

struct bf16_t { uint16_t v; };

__device__ __forceinline__ float bf_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {   // one v_cvt_pk_bf16_f32 (round to nearest even)
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

// A chunk is 16 bytes of a row: kV elements.
template <typename T> struct Chunk;
template <> struct Chunk<float> {
  static constexpr int kV = 4;
  static __device__ __forceinline__ void load(const float* p, float (&v)[4]) {
    const float4 q = *reinterpret_cast<const float4*>(p);
    v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
  }
  static __device__ __forceinline__ void store(float* p, const float (&v)[4]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  }
  static __device__ __forceinline__ void store_rounded(float* p, float (&v)[4]) { store(p, v); }
  static __device__ __forceinline__ void unpack(const uint4& q, float (&v)[4]) {
    v[0] = __uint_as_float(q.x); v[1] = __uint_as_float(q.y); v[2] = __uint_as_float(q.z); v[3] = __uint_as_float(q.w);
  }
};
template <> struct Chunk<bf16_t> {
  static constexpr int kV = 8;
  static __device__ __forceinline__ void load(const bf16_t* p, float (&v)[8]) {
    const uint4 q = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) { v[2 * j] = bf_lo(w[j]); v[2 * j + 1] = bf_hi(w[j]); }
  }
  static __device__ __forceinline__ void store(bf16_t* p, const float (&v)[8]) {
    *reinterpret_cast<uint4*>(p) = make_uint4(pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]), pack_bf16(v[4], v[5]), pack_bf16(v[6], v[7]));
  }
  static __device__ __forceinline__ void unpack(const uint4& q, float (&v)[8]) {
    const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) { v[2 * j] = bf_lo(w[j]); v[2 * j + 1] = bf_hi(w[j]); }
  }
  // stores v and leaves in v what a reader of p will find
  static __device__ __forceinline__ void store_rounded(bf16_t* p, float (&v)[8]) {
    const uint32_t w[4] = {pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]), pack_bf16(v[4], v[5]), pack_bf16(v[6], v[7])};
    *reinterpret_cast<uint4*>(p) = make_uint4(w[0], w[1], w[2], w[3]);
#pragma unroll
    for (int j = 0; j < 4; ++j) { v[2 * j] = bf_lo(w[j]); v[2 * j + 1] = bf_hi(w[j]); }
  }
};

__device__ __forceinline__ float ldw(const void* w, int wbf16, int i) {
  return wbf16 ? __uint_as_float((uint32_t)static_cast<const uint16_t*>(w)[i] << 16) : static_cast<const float*>(w)[i];
}
// V weights from index i0 on (a multiple of V, the array 16-byte aligned), in the fewest loads
template <int V>
__device__ __forceinline__ void ldwv(const void* w, int wbf16, int i0, float (&o)[V]) {
  if (wbf16) {
    if constexpr (V == 8) {
      Chunk<bf16_t>::load(static_cast<const bf16_t*>(w) + i0, o);
    } else {
      const uint2 q = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(w) + i0);
      o[0] = bf_lo(q.x); o[1] = bf_hi(q.x); o[2] = bf_lo(q.y); o[3] = bf_hi(q.y);
    }
  } else {
#pragma unroll
    for (int h = 0; h < V / 4; ++h) {
      const float4 q = *reinterpret_cast<const float4*>(static_cast<const float*>(w) + i0 + 4 * h);
      o[4 * h] = q.x; o[4 * h + 1] = q.y; o[4 * h + 2] = q.z; o[4 * h + 3] = q.w;
    }
  }
}

// ------------------------------------------------------------------------------------ LayerNorm
// G lanes share a row (G a power of two, 4..64), lane g holds the chunks g, g + G, ... of it: at
// most kMaxChunks of them, all in registers, so the row is read once.  Mean first, then the sum of
// squared deviations (the data is at hand, and E[x^2] - mean^2 would cancel for rows far from zero).
constexpr int kLnThreads = 256;
constexpr int kMaxChunks = 8;

struct LnArgs {
  const void* x;
  const void* w;
  const void* b;
  void* y;
  int64_t rows;
  int C, wbf16;
  float eps;
  // with the residual update in front (RES): the rows normalised are xo = x * s[c] + r (+ r2), also written out
  const void *s, *r, *r2;
  void* xo;
};

template <typename T, int G, int NC, bool RES>
__global__ __launch_bounds__(kLnThreads) void m2d_layernorm_kernel(const LnArgs a) {
  constexpr int V = Chunk<T>::kV;
  const int lane_in_row = threadIdx.x & (G - 1);
  const int row_in_block = threadIdx.x / G;
  constexpr int kRows = kLnThreads / G;
  const int nchunks = a.C / V;
  const float inv_c = 1.f / (float)a.C;
  // this lane's share of weight and bias, kept for all its rows
  float wv[NC][V], bv[NC][V];
#pragma unroll
  for (int k = 0; k < NC; ++k) {
    const int c = lane_in_row + k * G;
#pragma unroll
    for (int j = 0; j < V; ++j) { wv[k][j] = 0.f; bv[k][j] = 0.f; }
    if (c < nchunks) {
      ldwv<V>(a.w, a.wbf16, c * V, wv[k]);
      ldwv<V>(a.b, a.wbf16, c * V, bv[k]);
    }
  }
  float sv[RES ? NC : 1][V];
  if constexpr (RES) {
#pragma unroll
    for (int k = 0; k < NC; ++k) {
      const int c = lane_in_row + k * G;
#pragma unroll
      for (int j = 0; j < V; ++j) sv[k][j] = 0.f;
      if (c < nchunks) ldwv<V>(a.s, a.wbf16, c * V, sv[k]);
    }
  }
  const T* X = static_cast<const T*>(a.x);
  const T* R = static_cast<const T*>(a.r);
  const T* R2 = static_cast<const T*>(a.r2);
  T* XO = static_cast<T*>(a.xo);
  T* Y = static_cast<T*>(a.y);
  for (int64_t row = (int64_t)blockIdx.x * kRows + row_in_block; row < a.rows; row += (int64_t)gridDim.x * kRows) {
    float v[NC][V];
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < NC; ++k) {
      const int c = lane_in_row + k * G;
      if (c < nchunks) {
        Chunk<T>::load(X + row * a.C + c * V, v[k]);
        if constexpr (RES) {   // the residual update, as m2d_scale_residual_kernel computes it; the norm sees what was stored
          float r[V];
          Chunk<T>::load(R + row * a.C + c * V, r);
          if (R2) {
            float r2[V];
            Chunk<T>::load(R2 + row * a.C + c * V, r2);
#pragma unroll
            for (int j = 0; j < V; ++j) r[j] += r2[j];
          }
#pragma unroll
          for (int j = 0; j < V; ++j) v[k][j] = __builtin_fmaf(v[k][j], sv[k][j], r[j]);
          Chunk<T>::store_rounded(XO + row * a.C + c * V, v[k]);
        }
      } else {
#pragma unroll
        for (int j = 0; j < V; ++j) v[k][j] = 0.f;
      }
#pragma unroll
      for (int j = 0; j < V; ++j) s += v[k][j];
    }
#pragma unroll
    for (int off = G >> 1; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
    const float mean = s * inv_c;
    float q = 0.f;
#pragma unroll
    for (int k = 0; k < NC; ++k) {
      const int c = lane_in_row + k * G;
      if (c < nchunks) {
#pragma unroll
        for (int j = 0; j < V; ++j) { const float d = v[k][j] - mean; q = __builtin_fmaf(d, d, q); }
      }
    }
#pragma unroll
    for (int off = G >> 1; off > 0; off >>= 1) q += __shfl_xor(q, off, 64);
    const float rstd = rsqrtf(q * inv_c + a.eps);
#pragma unroll
    for (int k = 0; k < NC; ++k) {
      const int c = lane_in_row + k * G;
      if (c < nchunks) {
        float o[V];
#pragma unroll
        for (int j = 0; j < V; ++j) o[j] = __builtin_fmaf((v[k][j] - mean) * rstd, wv[k][j], bv[k][j]);
        Chunk<T>::store(Y + row * a.C + c * V, o);
      }
    }
  }
}

template <typename T, int G, int NC, bool RES>
int launch_ln(const LnArgs& a, hipStream_t st) {
  constexpr int kRows = kLnThreads / G;
  int64_t blocks = (a.rows + kRows - 1) / kRows;
  if (blocks > 256 * 8) blocks = 256 * 8;   // grid-stride beyond that: the lane's weights are loaded once and serve several rows
  hipLaunchKernelGGL((m2d_layernorm_kernel<T, G, NC, RES>), dim3((unsigned)blocks), dim3(kLnThreads), 0, st, a);
  return hipGetLastError() == hipSuccess ? M2D_OK : M2D_ERR_HIP;
}

template <typename T, bool RES>
int run_ln(const LnArgs& a, hipStream_t st) {
  const int nchunks = a.C / Chunk<T>::kV;
  // the fewest lanes per row that keep a lane's share within kMaxChunks, but at least 4 chunks in
  // flight per row where the row is long enough
  if (nchunks <= 4) return launch_ln<T, 4, 1, RES>(a, st);
  if (nchunks <= 8) return launch_ln<T, 8, 1, RES>(a, st);
  if (nchunks <= 16) return launch_ln<T, 16, 1, RES>(a, st);
  if (nchunks <= 32) return launch_ln<T, 16, 2, RES>(a, st);
  if (nchunks <= 64) return launch_ln<T, 16, 4, RES>(a, st);
  if (nchunks <= 128) return launch_ln<T, 32, 4, RES>(a, st);
  if (nchunks <= 256) return launch_ln<T, 64, 4, RES>(a, st);
  return launch_ln<T, 64, kMaxChunks, RES>(a, st);
}

// ------------------------------------------------------------------ depthwise 3x3, channel-last
// y[b,h,w,c] = sum_{i,j} wt[c][i][j] x[b,h+i-1,w+j-1,c], zero padding.  A thread owns one chunk of
// channels and a strip of STRIP cells along W; the 3x3 window slides along the strip, so every
// output costs three 16-byte loads plus the strip's two extra columns, and the 9 x kV weights of
// the chunk stay in registers.  The kernel is bound by the number of loads: strips of 14 (which
// divide the model's widths 56, 28, 14) run 7 % faster than strips of 8, strips of 4 45 % slower.
constexpr int kDwThreads = 256;
constexpr int kDwAhead = 4;        // columns between a fetch and its first use (2: 52 us, 3: 50 us, 4: 48 us at 56x56x128, B=128)

struct DwArgs {
  const void* x;
  const void* w;    // (C, 1, 3, 3)
  void* y;
  int B, H, W, C, wbf16;
  int strips;       // strips per image row
};

template <typename T, int STRIP>
__global__ __launch_bounds__(kDwThreads) void m2d_dwconv3x3_kernel(const DwArgs a) {
  constexpr int V = Chunk<T>::kV;
  const int nchunks = a.C / V;
  const int64_t total = (int64_t)a.B * a.H * a.strips * nchunks;
  const int64_t gid = (int64_t)blockIdx.x * kDwThreads + threadIdx.x;
  if (gid >= total) return;
  const int c = (int)(gid % nchunks);
  int64_t rest = gid / nchunks;
  const int sidx = (int)(rest % a.strips);
  rest /= a.strips;
  const int h = (int)(rest % a.H);
  const int b = (int)(rest / a.H);
  // the 9 taps of the chunk's V channels are 9 V consecutive weights: fetched as 9 groups of V
  float wt[9][V];
  {
    float flat[9][V];   // flat[g][i] = weight number g V + i of the chunk = channel (g V + i) / 9, tap (g V + i) % 9
#pragma unroll
    for (int g = 0; g < 9; ++g) ldwv<V>(a.w, a.wbf16, (c * 9 + g) * V, flat[g]);
#pragma unroll
    for (int t = 0; t < 9; ++t)
#pragma unroll
      for (int j = 0; j < V; ++j) wt[t][j] = flat[(j * 9 + t) / V][(j * 9 + t) % V];
  }
  const T* X = static_cast<const T*>(a.x) + ((int64_t)b * a.H * a.W) * a.C + c * V;
  T* Y = static_cast<T*>(a.y) + ((int64_t)b * a.H * a.W) * a.C + c * V;
  const int w0 = sidx * STRIP;
  // Window: the 16-byte chunks of the cells (h+i-1, w-1 .. w+kDwAhead) as they come from memory, columns that
  // rotate with the step; column w+kDwAhead is fetched kDwAhead steps before its first use, so that a thread has
  // 3 kDwAhead loads in flight (with one column ahead and three waves per SIMD the kernel waited for memory half of
  // the time).  Unpacked at every use: the conversions are cheap next to the registers a float window costs.
  constexpr int NS = kDwAhead + 2;      // columns held
  uint4 win[3][NS];
  auto load_col = [&](int col, int slot) {
#pragma unroll
    for (int i = 0; i < 3; ++i) {
      const int hh = h + i - 1;
      win[i][slot] = make_uint4(0u, 0u, 0u, 0u);
      if (hh >= 0 && hh < a.H && col >= 0 && col < a.W)
        win[i][slot] = *reinterpret_cast<const uint4*>(X + ((int64_t)hh * a.W + col) * a.C);
    }
  };
#pragma unroll
  for (int k = 0; k <= kDwAhead; ++k) load_col(w0 - 1 + k, k);
#pragma unroll
  for (int s = 0; s < STRIP; ++s) {
    const int w = w0 + s;
    if (w >= a.W) break;
    const int sl = s % NS, sm = (s + 1) % NS, sr = (s + 2) % NS;      // slots of columns w-1, w, w+1
    if (s + kDwAhead <= STRIP) load_col(w + kDwAhead, (s + kDwAhead + 1) % NS);
    float o[V];
#pragma unroll
    for (int j = 0; j < V; ++j) o[j] = 0.f;
#pragma unroll
    for (int i = 0; i < 3; ++i) {
      float xl[V], xm[V], xr[V];
      Chunk<T>::unpack(win[i][sl], xl);
      Chunk<T>::unpack(win[i][sm], xm);
      Chunk<T>::unpack(win[i][sr], xr);
#pragma unroll
      for (int j = 0; j < V; ++j) {
        o[j] = __builtin_fmaf(wt[3 * i][j], xl[j], o[j]);
        o[j] = __builtin_fmaf(wt[3 * i + 1][j], xm[j], o[j]);
        o[j] = __builtin_fmaf(wt[3 * i + 2][j], xr[j], o[j]);
      }
    }
    Chunk<T>::store(Y + ((int64_t)h * a.W + w) * a.C, o);
  }
}

// ------------------------------------------------------------------------ fused elementwise
// StarReLU, y = scale * relu(x)^2 + bias with scalar scale and bias (models/utils.py:22-37), and the
// residual update of a block, y = x * scale[c] + r (models/mamba2d.py:258-259), with a second branch
// r2 where the token mixer's answer is itself a sum (models/mamba2d.py:176): one pass each where stock
// operators take three and two or three.
constexpr int kEwThreads = 256;

struct EwArgs {
  const void* x;
  const void* r;      // residual branch (scale-residual only)
  const void* r2;     // second branch, or null (scale-residual only)
  const void* s;      // one scale (StarReLU) or C of them
  const void* b;      // one bias (StarReLU)
  void* y;
  int64_t chunks;     // 16-byte chunks in all
  int cpr;            // chunks per row (scale-residual)
  int wbf16;
};

template <typename T>
__global__ __launch_bounds__(kEwThreads) void m2d_starrelu_kernel(const EwArgs a) {
  constexpr int V = Chunk<T>::kV;
  const float sc = ldw(a.s, a.wbf16, 0), bi = ldw(a.b, a.wbf16, 0);
  const T* X = static_cast<const T*>(a.x);
  T* Y = static_cast<T*>(a.y);
  for (int64_t i = (int64_t)blockIdx.x * kEwThreads + threadIdx.x; i < a.chunks; i += (int64_t)gridDim.x * kEwThreads) {
    float v[V];
    Chunk<T>::load(X + i * V, v);
#pragma unroll
    for (int j = 0; j < V; ++j) { const float t = fmaxf(v[j], 0.f); v[j] = __builtin_fmaf(sc * t, t, bi); }
    Chunk<T>::store(Y + i * V, v);
  }
}

template <typename T>
__global__ __launch_bounds__(kEwThreads) void m2d_scale_residual_kernel(const EwArgs a) {
  constexpr int V = Chunk<T>::kV;
  const T* X = static_cast<const T*>(a.x);
  const T* R = static_cast<const T*>(a.r);
  const T* R2 = static_cast<const T*>(a.r2);
  T* Y = static_cast<T*>(a.y);
  for (int64_t i = (int64_t)blockIdx.x * kEwThreads + threadIdx.x; i < a.chunks; i += (int64_t)gridDim.x * kEwThreads) {
    const int c = (int)(i % a.cpr);
    float v[V], r[V];
    Chunk<T>::load(X + i * V, v);
    Chunk<T>::load(R + i * V, r);
    if (R2) {
      float r2[V];
      Chunk<T>::load(R2 + i * V, r2);
#pragma unroll
      for (int j = 0; j < V; ++j) r[j] += r2[j];
    }
    float sc[V];
    ldwv<V>(a.s, a.wbf16, c * V, sc);
#pragma unroll
    for (int j = 0; j < V; ++j) v[j] = __builtin_fmaf(v[j], sc[j], r[j]);
    Chunk<T>::store(Y + i * V, v);
  }
}

inline unsigned ew_blocks(int64_t chunks) {
  int64_t blocks = (chunks + kEwThreads - 1) / kEwThreads;
  return (unsigned)(blocks > 256 * 64 ? 256 * 64 : blocks);
}

// ------------------------------------------------------- rotary embedding + LayerNorm of q and k
// The attention stages rotate q and k by position (pairs of neighbouring features share an angle,
// models/utils.py:253-297) and then LayerNorm each head (:299-301).  Input is the output of the
// qkv projection, (B, L, 3, heads, hd); q and k leave as (B, heads, L, hd), the layout the attention
// kernel wants.  A head's hd features are G = hd / kV chunks on G neighbouring lanes; the pairs of
// the rotation never straddle a chunk.  One pass where stock operators take sixteen.
struct RopeArgs {
  const void* qkv;
  const void *cos, *sin;          // (L, hd), element type of qkv
  const void *qw, *qb, *kw, *kb;  // LayerNorm weights of q and k, (hd)
  void *q, *k;
  int64_t total;                  // B * L * 2 * heads * G chunks
  int L, heads, hd, wbf16;
  int token_major;                // q and k as (B, L, heads, hd) instead of (B, heads, L, hd)
  float eps;
};

template <typename T, int G>
__global__ __launch_bounds__(kEwThreads) void m2d_rope_qknorm_kernel(const RopeArgs a) {
  constexpr int V = Chunk<T>::kV;
  const int64_t gid = (int64_t)blockIdx.x * kEwThreads + threadIdx.x;
  if (gid >= a.total) return;          // whole groups of G lanes leave together (total is a multiple of G)
  const int c = (int)(gid % G);
  int64_t rest = gid / G;
  const int head = (int)(rest % a.heads);
  rest /= a.heads;
  const int which = (int)(rest % 2);   // 0: q, 1: k
  rest /= 2;
  const int l = (int)(rest % a.L);
  const int64_t b = rest / a.L;
  const T* src = static_cast<const T*>(a.qkv) + (((b * a.L + l) * 3 + which) * a.heads + head) * (int64_t)a.hd + c * V;
  float x[V], cs[V], sn[V];
  Chunk<T>::load(src, x);
  Chunk<T>::load(static_cast<const T*>(a.cos) + (int64_t)l * a.hd + c * V, cs);
  Chunk<T>::load(static_cast<const T*>(a.sin) + (int64_t)l * a.hd + c * V, sn);
  float v[V];
#pragma unroll
  for (int j = 0; j < V; j += 2) {
    v[j] = __builtin_fmaf(x[j], cs[j], -x[j + 1] * sn[j]);
    v[j + 1] = __builtin_fmaf(x[j + 1], cs[j + 1], x[j] * sn[j + 1]);
  }
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < V; ++j) s += v[j];
#pragma unroll
  for (int off = G >> 1; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
  const float inv = 1.f / (float)a.hd;
  const float mean = s * inv;
  float q = 0.f;
#pragma unroll
  for (int j = 0; j < V; ++j) { const float d = v[j] - mean; q = __builtin_fmaf(d, d, q); }
#pragma unroll
  for (int off = G >> 1; off > 0; off >>= 1) q += __shfl_xor(q, off, 64);
  const float rstd = rsqrtf(q * inv + a.eps);
  const void* w = which ? a.kw : a.qw;
  const void* bi = which ? a.kb : a.qb;
  float o[V], wv[V], bv[V];
  ldwv<V>(w, a.wbf16, c * V, wv);
  ldwv<V>(bi, a.wbf16, c * V, bv);
#pragma unroll
  for (int j = 0; j < V; ++j) o[j] = __builtin_fmaf((v[j] - mean) * rstd, wv[j], bv[j]);
  T* dst = static_cast<T*>(which ? a.k : a.q) +
           (a.token_major ? ((b * a.L + l) * a.heads + head) : ((b * a.heads + head) * a.L + l)) * (int64_t)a.hd + c * V;
  Chunk<T>::store(dst, o);
}

template <typename T>
int run_rope(const RopeArgs& a, int G, hipStream_t st) {
  const int64_t blocks = (a.total + kEwThreads - 1) / kEwThreads;
  if (blocks >= ((int64_t)1 << 31)) return M2D_ERR_UNSUPPORTED;
  const dim3 grid((unsigned)blocks), block(kEwThreads);
  switch (G) {
    case 1: hipLaunchKernelGGL((m2d_rope_qknorm_kernel<T, 1>), grid, block, 0, st, a); break;
    case 2: hipLaunchKernelGGL((m2d_rope_qknorm_kernel<T, 2>), grid, block, 0, st, a); break;
    case 4: hipLaunchKernelGGL((m2d_rope_qknorm_kernel<T, 4>), grid, block, 0, st, a); break;
    case 8: hipLaunchKernelGGL((m2d_rope_qknorm_kernel<T, 8>), grid, block, 0, st, a); break;
    case 16: hipLaunchKernelGGL((m2d_rope_qknorm_kernel<T, 16>), grid, block, 0, st, a); break;
    case 32: hipLaunchKernelGGL((m2d_rope_qknorm_kernel<T, 32>), grid, block, 0, st, a); break;
    default: return M2D_ERR_UNSUPPORTED;
  }
  return hipGetLastError() == hipSuccess ? M2D_OK : M2D_ERR_HIP;
}

// ---------------------------------------------------------------- small linear layers, bf16
// y = post(pre(x) W^T + bias) for the narrow layers of a block (K and N up to 512): in_proj, out_proj,
// the pointwise convolutions of the local path and the MLP at 64 or 128 channels
// (models/mamba2d.py:166-176, models/utils.py:58-81, 87-118).  These products are bandwidth-bound: a row
// of x is 128 to 512 bytes and is used once.  The weight matrix lives in LDS as bf16 for the whole
// (persistent) workgroup; a wave owns 16 rows, whose 16-byte pieces are the A operands of
// v_mfma_f32_16x16x32_bf16 as they come from memory (lane l: row l & 15, columns 8 (l >> 4) + j of a step
// of 32), W's rows are the B operands (lane l: output l & 15, the same columns), results leave through a
// per-wave LDS block so that memory sees 16-byte pieces of rows.  pre and post are nothing, GELU (exact
// form, through erf) or StarReLU: the activation that the block applies before or after the layer.
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ f32x4_t mfma_bf16(uint4 a, uint4 b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}
__device__ __forceinline__ uint4 ld16(const void* p) { return *reinterpret_cast<const uint4*>(p); }

constexpr int kLinThreads = 256;
constexpr int kLinWaves = 4;
constexpr int kLinStage = 72;      // floats per row of a wave's result block: 64 + 8
constexpr int kLinMaxKC = 16;      // steps of 32 along K: K <= 512
enum { kActNone = 0, kActGelu = 1, kActStarRelu = 2, kActLayerNorm = 3 };   // the last one only before the layer, and only inside this file

// erf by Abramowitz & Stegun 7.1.26 (absolute error below 1.5e-7), one v_exp_f32 and one v_rcp_f32
__device__ __forceinline__ float gelu_exact(float v) {
  const float z = fabsf(v) * 0.70710678118654752f;
  const float t = __builtin_amdgcn_rcpf(__builtin_fmaf(0.3275911f, z, 1.f));
  float poly = __builtin_fmaf(t, 1.061405429f, -1.453152027f);
  poly = __builtin_fmaf(t, poly, 1.421413741f);
  poly = __builtin_fmaf(t, poly, -0.284496736f);
  poly = __builtin_fmaf(t, poly, 0.254829592f);
  const float e = 1.f - poly * t * __builtin_amdgcn_exp2f(-z * z * 1.44269504088896341f);   // erf(|v| / sqrt 2)
  return 0.5f * v + 0.5f * fabsf(v) * e;                                                   // v erf(v/sqrt 2) = |v| erf(|v|/sqrt 2)
}
__device__ __forceinline__ float act(int kind, float v, float s, float b) {
  if (kind == kActGelu) return gelu_exact(v);
  if (kind == kActStarRelu) { const float t = fmaxf(v, 0.f); return __builtin_fmaf(s * t, t, b); }
  return v;
}

// LayerNorm of the 16 rows a wave holds as MFMA operands (lane (mn, kb): the 8 values at 32 kc + 8 kb + j of row
// mn, for kc < KC), in place, rounded to bf16 as a LayerNorm kernel in front of the layer would store them.
// lnp: weight then bias, K floats each, in LDS.  Two-pass mean / variance; the four lanes of a row meet through
// two lane exchanges.
template <int KCMAX>
__device__ __forceinline__ void norm_rows(uint4 (&A)[KCMAX], int KC, int K, const float* lnp, float eps, int kb) {
  float v[KCMAX][8];
  float s = 0.f;
#pragma unroll
  for (int kc = 0; kc < KCMAX; ++kc) {
    Chunk<bf16_t>::unpack(A[kc], v[kc]);
    if (kc < KC) {
#pragma unroll
      for (int j = 0; j < 8; ++j) s += v[kc][j];
    }
  }
  s += __shfl_xor(s, 16, 64);
  s += __shfl_xor(s, 32, 64);
  const float inv = 1.f / (float)K, mean = s * inv;
  float q = 0.f;
#pragma unroll
  for (int kc = 0; kc < KCMAX; ++kc)
    if (kc < KC) {
#pragma unroll
      for (int j = 0; j < 8; ++j) { const float d = v[kc][j] - mean; q = __builtin_fmaf(d, d, q); }
    }
  q += __shfl_xor(q, 16, 64);
  q += __shfl_xor(q, 32, 64);
  const float rstd = rsqrtf(q * inv + eps);
#pragma unroll
  for (int kc = 0; kc < KCMAX; ++kc)
    if (kc < KC) {
      const float* w = lnp + 32 * kc + 8 * kb;
      const float4 w0 = *reinterpret_cast<const float4*>(w), w1 = *reinterpret_cast<const float4*>(w + 4);
      const float4 b0 = *reinterpret_cast<const float4*>(w + K), b1 = *reinterpret_cast<const float4*>(w + K + 4);
      const float wv[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w}, bv[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
      float o[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = __builtin_fmaf((v[kc][j] - mean) * rstd, wv[j], bv[j]);
      A[kc] = make_uint4(pack_bf16(o[0], o[1]), pack_bf16(o[2], o[3]), pack_bf16(o[4], o[5]), pack_bf16(o[6], o[7]));
    }
}

struct LinArgs {
  const void* x;        // (P, K) bf16
  const void* w;        // (N, K)
  const void* bias;     // (N) or null
  void* y;              // (P, N) bf16
  int64_t P;
  int K, N, wbf16, pre, post, ntiles;
  int nsplit, Ns;       // the workgroups share out the N outputs in nsplit slices of Ns
  const void *pre_s, *pre_b, *post_s, *post_b;   // StarReLU scale and bias (one element each, type of w) where pre / post is StarReLU
  const void *ln_w, *ln_b;                       // LayerNorm over the K inputs in front of the layer (pre == kActLayerNorm): weight and bias, (K), type of w
  float ln_eps;
};

template <int KCMAX>   // steps of 32 along K that the kernel is built for: 2, 4, 8 or 16
__global__ __launch_bounds__(kLinThreads) void m2d_linear_kernel(const LinArgs a) {
  extern __shared__ float smem[];
  const int tid = threadIdx.x, l = tid & 63, mn = l & 15, kb = l >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ws = a.K + 8;                                // bf16 per row of W in LDS: rows stay 16-byte aligned and spread over the banks
  uint16_t* wl = reinterpret_cast<uint16_t*>(smem);
  float* stage = smem + (a.Ns * ws / 2 + 3) / 4 * 4 + wave * 16 * kLinStage;
  const int slice = blockIdx.x % a.nsplit, nbase = slice * a.Ns;   // this workgroup's outputs: nbase .. nbase + Ns
  const int first_tile = blockIdx.x / a.nsplit, tile_step = gridDim.x / a.nsplit;
  for (int i = tid; i < a.Ns * (a.K / 8); i += kLinThreads) {
    const int n = i / (a.K / 8), k8 = i - n * (a.K / 8);
    uint4 q;
    if (a.wbf16) {
      q = ld16(static_cast<const uint16_t*>(a.w) + (int64_t)(nbase + n) * a.K + 8 * k8);
    } else {
      const float* src = static_cast<const float*>(a.w) + (int64_t)(nbase + n) * a.K + 8 * k8;
      q = make_uint4(pack_bf16(src[0], src[1]), pack_bf16(src[2], src[3]), pack_bf16(src[4], src[5]), pack_bf16(src[6], src[7]));
    }
    *reinterpret_cast<uint4*>(wl + n * ws + 8 * k8) = q;
  }
  float* lnp = smem + (a.Ns * ws / 2 + 3) / 4 * 4 + kLinWaves * 16 * kLinStage;      // behind the waves' result blocks
  if (a.pre == kActLayerNorm)
    for (int i = tid; i < a.K; i += kLinThreads) { lnp[i] = ldw(a.ln_w, a.wbf16, i); lnp[a.K + i] = ldw(a.ln_b, a.wbf16, i); }
  __syncthreads();
  const float pre_s = a.pre == kActStarRelu ? ldw(a.pre_s, a.wbf16, 0) : 0.f, pre_b = a.pre == kActStarRelu ? ldw(a.pre_b, a.wbf16, 0) : 0.f;
  const float post_s = a.post == kActStarRelu ? ldw(a.post_s, a.wbf16, 0) : 0.f, post_b = a.post == kActStarRelu ? ldw(a.post_b, a.wbf16, 0) : 0.f;
  const int KC = a.K / 32;
  const uint16_t* X = static_cast<const uint16_t*>(a.x);
  uint16_t* Y = static_cast<uint16_t*>(a.y);
  // The rows of the next tile are fetched while the current one is worked on: with the weights in LDS
  // few waves fit a compute unit, too few to cover the latency of memory by themselves.
  uint4 Anext[KCMAX];
  auto fetch = [&](int tile) {
    const int64_t q0 = (int64_t)tile * 64 + wave * 16;
#pragma unroll
    for (int kc = 0; kc < KCMAX; ++kc) {
      Anext[kc] = make_uint4(0u, 0u, 0u, 0u);
      if (kc < KC && tile < a.ntiles && q0 + mn < a.P) Anext[kc] = ld16(X + (q0 + mn) * a.K + 32 * kc + 8 * kb);
    }
  };
  fetch(first_tile);
  for (int tile = first_tile; tile < a.ntiles; tile += tile_step) {
    const int64_t p0 = (int64_t)tile * 64 + wave * 16;
    const int rows = (int)(a.P - p0 < 16 ? a.P - p0 : 16);     // rows of the wave inside the array (may be <= 0)
    uint4 A[KCMAX];
#pragma unroll
    for (int kc = 0; kc < KCMAX; ++kc) A[kc] = Anext[kc];
    fetch(tile + tile_step);
    if (a.pre == kActLayerNorm) {   // (uniform; the host only asks for it where K <= 128)
      if constexpr (KCMAX <= 4) norm_rows<KCMAX>(A, KC, a.K, lnp, a.ln_eps, kb);
    } else if (a.pre != kActNone) {   // (uniform)
#pragma unroll
      for (int kc = 0; kc < KCMAX; ++kc)
        if (kc < KC) {
          uint32_t w4[4] = {A[kc].x, A[kc].y, A[kc].z, A[kc].w};
#pragma unroll
          for (int j = 0; j < 4; ++j)
            w4[j] = pack_bf16(act(a.pre, bf_lo(w4[j]), pre_s, pre_b), act(a.pre, bf_hi(w4[j]), pre_s, pre_b));
          A[kc] = make_uint4(w4[0], w4[1], w4[2], w4[3]);
        }
    }
    for (int n0 = 0; n0 < a.Ns; n0 += 64) {
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) {
        const int n = n0 + 16 * nt + mn;
        f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
        if (n0 + 16 * nt < a.Ns) {   // (uniform)
          const uint16_t* wrow = wl + n * ws + 8 * kb;
#pragma unroll
          for (int kc = 0; kc < KCMAX; ++kc)
            if (kc < KC) acc = mfma_bf16(A[kc], ld16(wrow + 32 * kc), acc);
          const float bn = a.bias ? ldw(a.bias, a.wbf16, nbase + n) : 0.f;
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[i] = act(a.post, acc[i] + bn, post_s, post_b);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) stage[(4 * kb + i) * kLinStage + 16 * nt + mn] = acc[i];   // position 4 kb + i, output 16 nt + mn
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
      for (int k = 0; k < 2; ++k) {   // the block's 16 x 8 pieces of 8 outputs, two per lane
        const int piece = l + 64 * k, c = piece >> 3, c8 = 8 * (piece & 7);
        if (c < rows && n0 + c8 < a.Ns) {
          const float4 lo = *reinterpret_cast<const float4*>(stage + c * kLinStage + c8);
          const float4 hi = *reinterpret_cast<const float4*>(stage + c * kLinStage + c8 + 4);
          *reinterpret_cast<uint4*>(Y + (p0 + c) * a.N + nbase + n0 + c8) =
              make_uint4(pack_bf16(lo.x, lo.y), pack_bf16(lo.z, lo.w), pack_bf16(hi.x, hi.y), pack_bf16(hi.z, hi.w));
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
  }
}

// ------------------------------------------------------------ the MLP of a narrow stage, bf16
// y = fc2(GELU(fc1 x)) (models/utils.py:58-81) where both weight matrices fit LDS together (C = 32 or 64
// channels, 4 C hidden units): the hidden activations, four times the size of x and y and the reason why
// the two layers run at the speed of memory writes when they are separate kernels, never leave the
// registers.  A wave owns 16 rows.  H^T = W1 X^T puts, in lane (mn, kb), the hidden units 16 nt + 4 kb + i of
// row mn; Y^T = W2 H^T contracts 32 hidden units per instruction and, as its operands may list them in any
// order as long as both agree, takes for the lane's eight slots exactly the units the lane holds (4 kb + i of
// two neighbouring tiles), with W2's rows read to match: no exchange of H between lanes.  Y^T leaves lane
// (mn, kb) with outputs 16 no + 4 kb + i of row mn: 8-byte stores.
struct MlpArgs {
  const void* x;          // (P, C) bf16
  const void *w1, *b1;    // (H, C), (H) or null
  const void *w2, *b2;    // (C, H), (C) or null
  void* y;                // (P, C) bf16
  int64_t P;
  int wbf16, ntiles;
  const void *ln_w, *ln_b;   // LayerNorm over C in front of fc1: weight and bias, (C), or null
  float ln_eps;
};

template <int KC>   // C = 32 KC channels, 128 KC hidden units
__global__ __launch_bounds__(kLinThreads) void m2d_mlp_kernel(const MlpArgs a) {
  constexpr int C = 32 * KC, HD = 4 * C, NH = HD / 16, NO = C / 16, NP = NH / 2;
  constexpr int W1S = C + 8;      // bf16 per row of W1 in LDS (a row per hidden unit)
  constexpr int W2S = HD + 4;     // bf16 per row of W2 (a row per output): rows stay 8-byte aligned and spread over the banks
  extern __shared__ float smem[];
  uint16_t* w1l = reinterpret_cast<uint16_t*>(smem);
  uint16_t* w2l = w1l + HD * W1S;
  float* b1l = reinterpret_cast<float*>(w2l + C * W2S);
  const int tid = threadIdx.x, l = tid & 63, mn = l & 15, kb = l >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  auto stage_weights = [&](const void* w, int rows, int cols, uint16_t* dst, int stride) {   // 8 elements at a time
    for (int i = tid; i < rows * (cols / 8); i += kLinThreads) {
      const int n = i / (cols / 8), k8 = i - n * (cols / 8);
      if (a.wbf16) {
        const uint4 q = ld16(static_cast<const uint16_t*>(w) + (int64_t)n * cols + 8 * k8);
        uint2* d = reinterpret_cast<uint2*>(dst + n * stride + 8 * k8);      // rows of W2 are 8-byte aligned only
        d[0] = make_uint2(q.x, q.y);
        d[1] = make_uint2(q.z, q.w);
      } else {
        const float* src = static_cast<const float*>(w) + (int64_t)n * cols + 8 * k8;
        uint2* d = reinterpret_cast<uint2*>(dst + n * stride + 8 * k8);
        d[0] = make_uint2(pack_bf16(src[0], src[1]), pack_bf16(src[2], src[3]));
        d[1] = make_uint2(pack_bf16(src[4], src[5]), pack_bf16(src[6], src[7]));
      }
    }
  };
  stage_weights(a.w1, HD, C, w1l, W1S);
  stage_weights(a.w2, C, HD, w2l, W2S);
  for (int i = tid; i < HD; i += kLinThreads) b1l[i] = a.b1 ? ldw(a.b1, a.wbf16, i) : 0.f;
  float* lnp = b1l + HD;
  if (a.ln_w)
    for (int i = tid; i < C; i += kLinThreads) { lnp[i] = ldw(a.ln_w, a.wbf16, i); lnp[C + i] = ldw(a.ln_b, a.wbf16, i); }
  float b2v[NO][4];
#pragma unroll
  for (int no = 0; no < NO; ++no)
#pragma unroll
    for (int i = 0; i < 4; ++i) b2v[no][i] = a.b2 ? ldw(a.b2, a.wbf16, 16 * no + 4 * kb + i) : 0.f;
  __syncthreads();
  const uint16_t* X = static_cast<const uint16_t*>(a.x);
  uint16_t* Y = static_cast<uint16_t*>(a.y);
  const f32x4_t zero = {0.f, 0.f, 0.f, 0.f};
  uint4 Xnext[KC];
  auto fetch = [&](int tile) {
    const int64_t q0 = (int64_t)tile * 64 + wave * 16;
#pragma unroll
    for (int kc = 0; kc < KC; ++kc) {
      Xnext[kc] = make_uint4(0u, 0u, 0u, 0u);
      if (tile < a.ntiles && q0 + mn < a.P) Xnext[kc] = ld16(X + (q0 + mn) * C + 32 * kc + 8 * kb);
    }
  };
  fetch(blockIdx.x);
  for (int tile = blockIdx.x; tile < a.ntiles; tile += gridDim.x) {
    const int64_t p0 = (int64_t)tile * 64 + wave * 16;
    uint4 Xf[KC];
#pragma unroll
    for (int kc = 0; kc < KC; ++kc) Xf[kc] = Xnext[kc];
    fetch(tile + gridDim.x);
    if (a.ln_w) norm_rows<KC>(Xf, KC, C, lnp, a.ln_eps, kb);      // (uniform)
    f32x4_t h[NH];
#pragma unroll
    for (int nt = 0; nt < NH; ++nt) {
      f32x4_t acc = zero;
#pragma unroll
      for (int kc = 0; kc < KC; ++kc) acc = mfma_bf16(ld16(w1l + (16 * nt + mn) * W1S + 32 * kc + 8 * kb), Xf[kc], acc);
      const float4 b1 = *reinterpret_cast<const float4*>(b1l + 16 * nt + 4 * kb);
      h[nt][0] = gelu_exact(acc[0] + b1.x);
      h[nt][1] = gelu_exact(acc[1] + b1.y);
      h[nt][2] = gelu_exact(acc[2] + b1.z);
      h[nt][3] = gelu_exact(acc[3] + b1.w);
    }
    uint4 hf[NP];      // the hidden activations as bf16, as fc2 of the stock path would read them
#pragma unroll
    for (int ks = 0; ks < NP; ++ks)
      hf[ks] = make_uint4(pack_bf16(h[2 * ks][0], h[2 * ks][1]), pack_bf16(h[2 * ks][2], h[2 * ks][3]),
                          pack_bf16(h[2 * ks + 1][0], h[2 * ks + 1][1]), pack_bf16(h[2 * ks + 1][2], h[2 * ks + 1][3]));
#pragma unroll
    for (int no = 0; no < NO; ++no) {
      f32x4_t acc = zero;
#pragma unroll
      for (int ks = 0; ks < NP; ++ks) {
        const uint16_t* w = w2l + (16 * no + mn) * W2S + 32 * ks + 4 * kb;      // output 16 no + mn, units 32 ks + 4 kb + {0..3, 16..19}
        const uint2 lo = *reinterpret_cast<const uint2*>(w), hi = *reinterpret_cast<const uint2*>(w + 16);
        acc = mfma_bf16(make_uint4(lo.x, lo.y, hi.x, hi.y), hf[ks], acc);
      }
      if (p0 + mn < a.P)
        *reinterpret_cast<uint2*>(Y + (p0 + mn) * C + 16 * no + 4 * kb) =
            make_uint2(pack_bf16(acc[0] + b2v[no][0], acc[1] + b2v[no][1]), pack_bf16(acc[2] + b2v[no][2], acc[3] + b2v[no][3]));
    }
  }
}

template <int KC>
constexpr size_t mlp_lds_bytes() { return (size_t)(128 * KC) * (32 * KC + 8) * 2 + (size_t)(32 * KC) * (128 * KC + 4) * 2 + (size_t)(128 * KC) * 4 + (size_t)(64 * KC) * 4; }

constexpr size_t kLinMaxLds = 160 * 1024;   // LDS of a compute unit

// More than 64 KB of dynamic LDS has to be allowed per kernel and device, once.
inline bool allow_big_lds() {
  static std::atomic<uint64_t> seen{0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return false;
  const uint64_t bit = 1ull << (dev & 63);
  if (seen.load(std::memory_order_acquire) & bit) return true;
  const void* kernels[] = {reinterpret_cast<const void*>(&m2d_linear_kernel<2>), reinterpret_cast<const void*>(&m2d_linear_kernel<4>),
                           reinterpret_cast<const void*>(&m2d_linear_kernel<8>), reinterpret_cast<const void*>(&m2d_linear_kernel<16>),
                           reinterpret_cast<const void*>(&m2d_mlp_kernel<1>), reinterpret_cast<const void*>(&m2d_mlp_kernel<2>)};
  for (const void* k : kernels)
    if (hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLinMaxLds) != hipSuccess) return false;
  seen.fetch_or(bit, std::memory_order_release);
  return true;
}

inline size_t linear_lds_bytes(int K, int N, bool ln = false) {
  return ((size_t)N * (K + 8) / 2 + 3) / 4 * 4 * 4 + (size_t)kLinWaves * 16 * kLinStage * 4 + (ln ? (size_t)2 * K * 4 : 0);
}

inline bool misaligned(const void* p, size_t n) { return (reinterpret_cast<uintptr_t>(p) & (n - 1)) != 0; }

// ------------------------------------------ attention of the rotary stages, one head per workgroup
// softmax(q k^T / sqrt(hd)) v with q and k rotated by position and LayerNormed per head first
// (models/utils.py:253-316), for heads of 32 features and up to 256 tokens (the 14x14 and 7x7 grids of
// the attention stages), straight from the output of the qkv projection, (B, L, 3, heads, 32), to
// (B, L, heads, 32), the input of the output projection: one pass in place of the rotation, the two
// LayerNorms, the attention kernel and the copies between them.
//   staging: a quad of lanes rotates and normalises q and k of a token (8 features per lane) and leaves
//     them in LDS as bf16 rows, and v transposed (feature-major), rows and columns past L zero;
//   a wave takes 16 queries at a time.  S^T = K Q^T, one v_mfma_f32_16x16x32_bf16 per 16 keys (the
//     contraction is the 32 features): lane (mn, kb) holds the scores of query mn for keys 16 kt + 4 kb + i.
//     Row maximum and sum are in-lane plus two lane exchanges (kb).  O^T = V^T P^T contracts 32 keys per
//     instruction; its operands may list the keys in any order as long as both agree, so the lane's
//     eight slots take the probabilities it already holds (keys 4 kb + i of two neighbouring tiles) and
//     V^T supplies the same keys: no exchange of the probabilities between lanes.
constexpr int kAttHd = 32;
constexpr int kAttRow = kAttHd + 8;     // bf16 per row of q and k in LDS
constexpr int kAttMaxL = 256;

struct AttnArgs {
  const void* qkv;                 // (B, L, 3, heads, 32) bf16
  const void *cos, *sin;           // (L, 32) bf16
  const void *qw, *qb, *kw, *kb;   // LayerNorm weights of q and k, (32)
  void* out;                       // (B, L, heads, 32) bf16
  int L, heads, wbf16;
  float eps, scale_log2e;          // softmax scale times log2(e)
};

// sum over the four lanes of a quad (lanes 4 g .. 4 g + 3), left in all of them
__device__ __forceinline__ float quad_sum(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, true));   // quad_perm [1,0,3,2]
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, true));   // quad_perm [2,3,0,1]
  return v;
}

// A quarter (8 features, one lane of a quad) of one token's q or k: rotation, LayerNorm over the quad, bf16 to dst.
__device__ __forceinline__ void rope_norm_quarter(const uint16_t* src, const float (&cs)[8], const float (&sn)[8], const float (&wv)[8],
                                                  const float (&bv)[8], float eps, uint16_t* dst) {
  float x[8], v[8];
  Chunk<bf16_t>::load(reinterpret_cast<const bf16_t*>(src), x);
#pragma unroll
  for (int j = 0; j < 8; j += 2) {
    v[j] = __builtin_fmaf(x[j], cs[j], -x[j + 1] * sn[j]);
    v[j + 1] = __builtin_fmaf(x[j + 1], cs[j + 1], x[j] * sn[j + 1]);
  }
  const float mean = quad_sum(((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]))) * (1.f / kAttHd);
  float d[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) d[j] = v[j] - mean;
  const float sq = quad_sum(((d[0] * d[0] + d[1] * d[1]) + (d[2] * d[2] + d[3] * d[3])) + ((d[4] * d[4] + d[5] * d[5]) + (d[6] * d[6] + d[7] * d[7])));
  const float rstd = rsqrtf(sq * (1.f / kAttHd) + eps);
  float o[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) o[j] = __builtin_fmaf(d[j] * rstd, wv[j], bv[j]);
  *reinterpret_cast<uint4*>(dst) = make_uint4(pack_bf16(o[0], o[1]), pack_bf16(o[2], o[3]), pack_bf16(o[4], o[5]), pack_bf16(o[6], o[7]));
}

constexpr int att_waves(int nt) { return nt <= 4 ? nt : (nt + 1) / 2; }   // one or two tiles of 16 queries per wave

template <int NT>   // tiles of 16 tokens: 16 (NT - 1) < L <= 16 NT
__global__ __launch_bounds__(64 * att_waves(NT)) __attribute__((amdgpu_waves_per_eu(4, 8)))
void m2d_rope_attention_kernel(const AttnArgs a) {
  constexpr int NP = (NT + 1) / 2;      // steps of 32 keys in the second product
  constexpr int LQ = 16 * NT;           // rows of q and k
  constexpr int LP = 32 * NP;           // columns of V^T
  constexpr int VS = LP + 4;            // bf16 per row of V^T: rows stay 8-byte aligned and spread over the banks
  constexpr int kThreads = 64 * att_waves(NT);
  __shared__ __attribute__((aligned(16))) uint16_t Qs[LQ * kAttRow];
  __shared__ __attribute__((aligned(16))) uint16_t Ks[LQ * kAttRow];
  __shared__ __attribute__((aligned(16))) uint16_t Vt[kAttHd * VS];
  const int tid = threadIdx.x, l = tid & 63, mn = l & 15, kb = l >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int head = blockIdx.x % a.heads;
  const int64_t b = blockIdx.x / a.heads;
  const int part = a.heads * kAttHd;                     // elements from q to k to v of a token
  const uint16_t* base = static_cast<const uint16_t*>(a.qkv) + (b * a.L * 3 * a.heads + head) * (int64_t)kAttHd;
  {   // staging: a quad of lanes per token, 8 features each, so that a token's 64 bytes are one piece of a load
    const int c8 = 8 * (tid & 3);
    float wq[8], bq[8], wk[8], bk[8];
    ldwv<8>(a.qw, a.wbf16, c8, wq);
    ldwv<8>(a.qb, a.wbf16, c8, bq);
    ldwv<8>(a.kw, a.wbf16, c8, wk);
    ldwv<8>(a.kb, a.wbf16, c8, bk);
    for (int t = tid >> 2; t < LP; t += kThreads / 4) {
      uint16_t* qd = Qs + t * kAttRow + c8;
      uint16_t* kd = Ks + t * kAttRow + c8;
      if (t < a.L) {     // (whole quads take the same side)
        const uint16_t* row = base + (int64_t)t * 3 * part + c8;
        float cs[8], sn[8];
        Chunk<bf16_t>::load(static_cast<const bf16_t*>(a.cos) + t * kAttHd + c8, cs);
        Chunk<bf16_t>::load(static_cast<const bf16_t*>(a.sin) + t * kAttHd + c8, sn);
        const uint4 vq = ld16(row + 2 * part);
        rope_norm_quarter(row, cs, sn, wq, bq, a.eps, qd);
        rope_norm_quarter(row + part, cs, sn, wk, bk, a.eps, kd);
        const uint32_t w4[4] = {vq.x, vq.y, vq.z, vq.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          Vt[(c8 + 2 * j) * VS + t] = (uint16_t)(w4[j] & 0xffffu);
          Vt[(c8 + 2 * j + 1) * VS + t] = (uint16_t)(w4[j] >> 16);
        }
      } else {
        if (t < LQ) {
          *reinterpret_cast<uint4*>(qd) = make_uint4(0u, 0u, 0u, 0u);
          *reinterpret_cast<uint4*>(kd) = make_uint4(0u, 0u, 0u, 0u);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) Vt[(c8 + j) * VS + t] = 0;
      }
    }
  }
  __syncthreads();
  const float ninf = -__builtin_huge_valf();
  const f32x4_t zero = {0.f, 0.f, 0.f, 0.f};
  uint16_t* out = static_cast<uint16_t*>(a.out);
  for (int qt = wave; qt < NT; qt += att_waves(NT)) {
    // The operands from k and v are the same for both tiles of a wave; read again, they cost LDS cycles that are
    // free here, kept in registers they would cost a quarter of the waves.  An offset the compiler cannot see
    // through keeps the loads inside the loop.
    int again = 0;
    asm volatile("" : "+v"(again));
    const uint16_t* Kl = Ks + again;
    const uint16_t* Vl = Vt + again;
    const uint4 qf = ld16(Qs + (16 * qt + mn) * kAttRow + 8 * kb);
    f32x4_t s[NT];
#pragma unroll
    for (int kt = 0; kt < NT; ++kt) s[kt] = mfma_bf16(ld16(Kl + (16 * kt + mn) * kAttRow + 8 * kb), qf, zero);
#pragma unroll
    for (int i = 0; i < 4; ++i)      // only the last tile can hold keys past the end: they take no part
      if (16 * (NT - 1) + 4 * kb + i >= a.L) s[NT - 1][i] = ninf;
    // maximum and sum run as four chains (one per i) and meet at the end
    float mx[4] = {ninf, ninf, ninf, ninf};
#pragma unroll
    for (int kt = 0; kt < NT; ++kt)
#pragma unroll
      for (int i = 0; i < 4; ++i) mx[i] = fmaxf(mx[i], s[kt][i]);
    float m = fmaxf(fmaxf(mx[0], mx[1]), fmaxf(mx[2], mx[3]));
    m = fmaxf(m, __shfl_xor(m, 16, 64));
    m = fmaxf(m, __shfl_xor(m, 32, 64));
    const float mc = m * a.scale_log2e;
    float sm[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kt = 0; kt < NT; ++kt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float pr = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kt][i], a.scale_log2e, -mc));
        s[kt][i] = pr;
        sm[i] += pr;
      }
    float sum = (sm[0] + sm[1]) + (sm[2] + sm[3]);
    sum += __shfl_xor(sum, 16, 64);
    sum += __shfl_xor(sum, 32, 64);
    f32x4_t o0 = zero, o1 = zero;
#pragma unroll
    for (int ks = 0; ks < NP; ++ks) {
      uint4 pf;
      pf.x = pack_bf16(s[2 * ks][0], s[2 * ks][1]);
      pf.y = pack_bf16(s[2 * ks][2], s[2 * ks][3]);
      if (2 * ks + 1 < NT) {
        pf.z = pack_bf16(s[2 * ks + 1][0], s[2 * ks + 1][1]);
        pf.w = pack_bf16(s[2 * ks + 1][2], s[2 * ks + 1][3]);
      } else {      // an odd number of tiles: the last step holds 16 keys
        pf.z = 0u; pf.w = 0u;
      }
      const uint16_t* v0 = Vl + mn * VS + 32 * ks + 4 * kb;      // features mn and 16 + mn, keys 32 ks + 4 kb + {0..3, 16..19}
      const uint2 a0 = *reinterpret_cast<const uint2*>(v0), a1 = *reinterpret_cast<const uint2*>(v0 + 16);
      const uint2 c0 = *reinterpret_cast<const uint2*>(v0 + 16 * VS), c1 = *reinterpret_cast<const uint2*>(v0 + 16 * VS + 16);
      o0 = mfma_bf16(make_uint4(a0.x, a0.y, a1.x, a1.y), pf, o0);
      o1 = mfma_bf16(make_uint4(c0.x, c0.y, c1.x, c1.y), pf, o1);
    }
    const float inv = 1.f / sum;
    const int q = 16 * qt + mn;
    if (q < a.L) {      // lane (mn, kb): features 4 kb + i and 16 + 4 kb + i of query mn
      uint16_t* dst = out + ((b * a.L + q) * a.heads + head) * (int64_t)kAttHd + 4 * kb;
      *reinterpret_cast<uint2*>(dst) = make_uint2(pack_bf16(o0[0] * inv, o0[1] * inv), pack_bf16(o0[2] * inv, o0[3] * inv));
      *reinterpret_cast<uint2*>(dst + 16) = make_uint2(pack_bf16(o1[0] * inv, o1[1] * inv), pack_bf16(o1[2] * inv, o1[3] * inv));
    }
  }
}

template <int NT>
void launch_attention(const AttnArgs& a, unsigned blocks, hipStream_t st) {
  hipLaunchKernelGGL(m2d_rope_attention_kernel<NT>, dim3(blocks), dim3(64 * att_waves(NT)), 0, st, a);
}

}  // namespace

extern "C" {

int m2d_layernorm_fwd(int64_t rows, int C, int dtype, int weight_dtype, const void* x, const void* weight,
                      const void* bias, float eps, void* y, void* stream) {
  if (!x || !weight || !bias || !y) return M2D_ERR_NULL_POINTER;
  if (rows < 1 || C < 1) return M2D_ERR_BAD_SHAPE;
  if ((dtype != M2D_F32 && dtype != M2D_BF16) || (weight_dtype != M2D_F32 && weight_dtype != M2D_BF16)) return M2D_ERR_UNSUPPORTED;
  const int V = dtype == M2D_BF16 ? 8 : 4;
  if (C % V != 0 || C / V > 64 * kMaxChunks) return M2D_ERR_UNSUPPORTED;   // rows of whole 16-byte chunks, at most 4096 (bf16) / 2048 (fp32) channels
  if (misaligned(x, 16) || misaligned(y, 16) || misaligned(weight, 16) || misaligned(bias, 16)) return M2D_ERR_MISALIGNED;
  LnArgs a = {};
  a.x = x; a.w = weight; a.b = bias; a.y = y; a.rows = rows; a.C = C; a.wbf16 = weight_dtype == M2D_BF16; a.eps = eps;
  hipStream_t st = static_cast<hipStream_t>(stream);
  return dtype == M2D_F32 ? run_ln<float, false>(a, st) : run_ln<bf16_t, false>(a, st);
}

int m2d_scale_residual_layernorm_fwd(int64_t rows, int C, int dtype, int weight_dtype, const void* x, const void* scale,
                                     const void* residual, const void* residual2, const void* weight, const void* bias,
                                     float eps, void* x_out, void* y, void* stream) {
  if (!x || !scale || !residual || !weight || !bias || !x_out || !y) return M2D_ERR_NULL_POINTER;
  if (rows < 1 || C < 1) return M2D_ERR_BAD_SHAPE;
  if ((dtype != M2D_F32 && dtype != M2D_BF16) || (weight_dtype != M2D_F32 && weight_dtype != M2D_BF16)) return M2D_ERR_UNSUPPORTED;
  const int V = dtype == M2D_BF16 ? 8 : 4;
  if (C % V != 0 || C / V > 64 * kMaxChunks) return M2D_ERR_UNSUPPORTED;
  if (misaligned(x, 16) || misaligned(residual, 16) || misaligned(residual2, 16) || misaligned(x_out, 16) || misaligned(y, 16) ||
      misaligned(scale, 16) || misaligned(weight, 16) || misaligned(bias, 16))
    return M2D_ERR_MISALIGNED;
  LnArgs a = {};
  a.x = x; a.w = weight; a.b = bias; a.y = y; a.rows = rows; a.C = C; a.wbf16 = weight_dtype == M2D_BF16; a.eps = eps;
  a.s = scale; a.r = residual; a.r2 = residual2; a.xo = x_out;
  hipStream_t st = static_cast<hipStream_t>(stream);
  return dtype == M2D_F32 ? run_ln<float, true>(a, st) : run_ln<bf16_t, true>(a, st);
}

int m2d_dwconv3x3_fwd(int B, int H, int W, int C, int dtype, int weight_dtype, const void* x, const void* weight,
                      void* y, void* stream) {
  if (!x || !weight || !y) return M2D_ERR_NULL_POINTER;
  if (B < 1 || H < 1 || W < 1 || C < 1) return M2D_ERR_BAD_SHAPE;
  if ((dtype != M2D_F32 && dtype != M2D_BF16) || (weight_dtype != M2D_F32 && weight_dtype != M2D_BF16)) return M2D_ERR_UNSUPPORTED;
  const int V = dtype == M2D_BF16 ? 8 : 4;
  if (C % V != 0) return M2D_ERR_UNSUPPORTED;
  if (misaligned(x, 16) || misaligned(y, 16) || misaligned(weight, 16)) return M2D_ERR_MISALIGNED;
  DwArgs a;
  a.x = x; a.w = weight; a.y = y; a.B = B; a.H = H; a.W = W; a.C = C; a.wbf16 = weight_dtype == M2D_BF16;
  const int strip = W % 14 == 0 ? 14 : 8;
  a.strips = (W + strip - 1) / strip;
  const int64_t total = (int64_t)B * H * a.strips * (C / V);
  const int64_t blocks = (total + kDwThreads - 1) / kDwThreads;
  if (blocks >= ((int64_t)1 << 31)) return M2D_ERR_UNSUPPORTED;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)blocks), block(kDwThreads);
  if (dtype == M2D_F32) {
    if (strip == 14) hipLaunchKernelGGL((m2d_dwconv3x3_kernel<float, 14>), grid, block, 0, st, a);
    else hipLaunchKernelGGL((m2d_dwconv3x3_kernel<float, 8>), grid, block, 0, st, a);
  } else {
    if (strip == 14) hipLaunchKernelGGL((m2d_dwconv3x3_kernel<bf16_t, 14>), grid, block, 0, st, a);
    else hipLaunchKernelGGL((m2d_dwconv3x3_kernel<bf16_t, 8>), grid, block, 0, st, a);
  }
  return hipGetLastError() == hipSuccess ? M2D_OK : M2D_ERR_HIP;
}

int m2d_starrelu_fwd(int64_t n, int dtype, int weight_dtype, const void* x, const void* scale, const void* bias, void* y,
                     void* stream) {
  if (!x || !scale || !bias || !y) return M2D_ERR_NULL_POINTER;
  if (n < 1) return M2D_ERR_BAD_SHAPE;
  if ((dtype != M2D_F32 && dtype != M2D_BF16) || (weight_dtype != M2D_F32 && weight_dtype != M2D_BF16)) return M2D_ERR_UNSUPPORTED;
  const int V = dtype == M2D_BF16 ? 8 : 4;
  if (n % V != 0) return M2D_ERR_UNSUPPORTED;
  if (misaligned(x, 16) || misaligned(y, 16)) return M2D_ERR_MISALIGNED;
  EwArgs a = {};
  a.x = x; a.s = scale; a.b = bias; a.y = y; a.chunks = n / V; a.wbf16 = weight_dtype == M2D_BF16;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == M2D_F32) hipLaunchKernelGGL(m2d_starrelu_kernel<float>, dim3(ew_blocks(a.chunks)), dim3(kEwThreads), 0, st, a);
  else hipLaunchKernelGGL(m2d_starrelu_kernel<bf16_t>, dim3(ew_blocks(a.chunks)), dim3(kEwThreads), 0, st, a);
  return hipGetLastError() == hipSuccess ? M2D_OK : M2D_ERR_HIP;
}

int m2d_scale_residual_fwd(int64_t rows, int C, int dtype, int weight_dtype, const void* x, const void* scale,
                           const void* residual, const void* residual2, void* y, void* stream) {
  if (!x || !scale || !residual || !y) return M2D_ERR_NULL_POINTER;
  if (rows < 1 || C < 1) return M2D_ERR_BAD_SHAPE;
  if ((dtype != M2D_F32 && dtype != M2D_BF16) || (weight_dtype != M2D_F32 && weight_dtype != M2D_BF16)) return M2D_ERR_UNSUPPORTED;
  const int V = dtype == M2D_BF16 ? 8 : 4;
  if (C % V != 0) return M2D_ERR_UNSUPPORTED;
  if (misaligned(x, 16) || misaligned(residual, 16) || misaligned(residual2, 16) || misaligned(y, 16) || misaligned(scale, 16))
    return M2D_ERR_MISALIGNED;
  EwArgs a = {};
  a.x = x; a.r = residual; a.r2 = residual2; a.s = scale; a.y = y; a.cpr = C / V; a.chunks = rows * a.cpr; a.wbf16 = weight_dtype == M2D_BF16;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == M2D_F32) hipLaunchKernelGGL(m2d_scale_residual_kernel<float>, dim3(ew_blocks(a.chunks)), dim3(kEwThreads), 0, st, a);
  else hipLaunchKernelGGL(m2d_scale_residual_kernel<bf16_t>, dim3(ew_blocks(a.chunks)), dim3(kEwThreads), 0, st, a);
  return hipGetLastError() == hipSuccess ? M2D_OK : M2D_ERR_HIP;
}

int m2d_rope_qknorm_fwd(int B, int L, int heads, int head_dim, int dtype, int weight_dtype, const void* qkv,
                        const void* cos, const void* sin, const void* q_weight, const void* q_bias, const void* k_weight,
                        const void* k_bias, float eps, int token_major, void* q, void* k, void* stream) {
  const void* req[] = {qkv, cos, sin, q_weight, q_bias, k_weight, k_bias, q, k};
  for (const void* p : req) if (!p) return M2D_ERR_NULL_POINTER;
  if (B < 1 || L < 1 || heads < 1 || head_dim < 1) return M2D_ERR_BAD_SHAPE;
  if ((dtype != M2D_F32 && dtype != M2D_BF16) || (weight_dtype != M2D_F32 && weight_dtype != M2D_BF16)) return M2D_ERR_UNSUPPORTED;
  const int V = dtype == M2D_BF16 ? 8 : 4;
  const int G = head_dim / V;
  if (head_dim % V != 0 || (G & (G - 1)) != 0 || G > 32) return M2D_ERR_UNSUPPORTED;   // a head is 1, 2, 4 ... 32 chunks
  for (const void* p : req) if (misaligned(p, 16)) return M2D_ERR_MISALIGNED;
  RopeArgs a = {};
  a.qkv = qkv; a.cos = cos; a.sin = sin; a.qw = q_weight; a.qb = q_bias; a.kw = k_weight; a.kb = k_bias; a.q = q; a.k = k;
  a.L = L; a.heads = heads; a.hd = head_dim; a.wbf16 = weight_dtype == M2D_BF16; a.eps = eps; a.token_major = token_major != 0;
  a.total = (int64_t)B * L * 2 * heads * G;
  hipStream_t st = static_cast<hipStream_t>(stream);
  return dtype == M2D_F32 ? run_rope<float>(a, G, st) : run_rope<bf16_t>(a, G, st);
}

int m2d_mlp_fwd(int64_t P, int C, int hidden, int weight_dtype, const void* x, const void* ln_weight, const void* ln_bias, float eps,
                const void* w1, const void* b1, const void* w2, const void* b2, void* y, void* stream) {
  if (!x || !w1 || !w2 || !y || (ln_weight != nullptr) != (ln_bias != nullptr)) return M2D_ERR_NULL_POINTER;
  if (P < 1 || C < 1 || hidden < 1) return M2D_ERR_BAD_SHAPE;
  if (weight_dtype != M2D_F32 && weight_dtype != M2D_BF16) return M2D_ERR_UNSUPPORTED;
  if ((C != 32 && C != 64) || hidden != 4 * C) return M2D_ERR_UNSUPPORTED;
  if ((P + 63) / 64 >= ((int64_t)1 << 31)) return M2D_ERR_UNSUPPORTED;
  if (misaligned(x, 16) || misaligned(y, 16) || misaligned(w1, 16) || misaligned(w2, 16) || (b1 && misaligned(b1, 4)) || (b2 && misaligned(b2, 4)) ||
      (ln_weight && (misaligned(ln_weight, 4) || misaligned(ln_bias, 4))))
    return M2D_ERR_MISALIGNED;
  MlpArgs a = {};
  a.ln_w = ln_weight; a.ln_b = ln_bias; a.ln_eps = eps;
  a.x = x; a.w1 = w1; a.b1 = b1; a.w2 = w2; a.b2 = b2; a.y = y; a.P = P; a.wbf16 = weight_dtype == M2D_BF16;
  a.ntiles = (int)((P + 63) / 64);
  const size_t lds = C == 64 ? mlp_lds_bytes<2>() : mlp_lds_bytes<1>();
  if (lds > 64 * 1024 && !allow_big_lds()) return M2D_ERR_HIP;
  int per_cu = (int)(160 * 1024 / lds);      // persistent: the weights go to LDS once per workgroup
  if (per_cu > 4) per_cu = 4;
  int grid = 256 * per_cu;
  if (grid > a.ntiles) grid = a.ntiles;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (C == 64) hipLaunchKernelGGL(m2d_mlp_kernel<2>, dim3((unsigned)grid), dim3(kLinThreads), lds, st, a);
  else hipLaunchKernelGGL(m2d_mlp_kernel<1>, dim3((unsigned)grid), dim3(kLinThreads), lds, st, a);
  return hipGetLastError() == hipSuccess ? M2D_OK : M2D_ERR_HIP;
}

int m2d_rope_attention_fwd(int B, int L, int heads, int head_dim, int weight_dtype, const void* qkv, const void* cos,
                           const void* sin, const void* q_weight, const void* q_bias, const void* k_weight,
                           const void* k_bias, float eps, float scale, void* out, void* stream) {
  if (!qkv || !cos || !sin || !q_weight || !q_bias || !k_weight || !k_bias || !out) return M2D_ERR_NULL_POINTER;
  if (B < 1 || L < 1 || heads < 1) return M2D_ERR_BAD_SHAPE;
  if (weight_dtype != M2D_F32 && weight_dtype != M2D_BF16) return M2D_ERR_UNSUPPORTED;
  if (head_dim != kAttHd || L > kAttMaxL) return M2D_ERR_UNSUPPORTED;
  if ((int64_t)B * heads >= ((int64_t)1 << 31)) return M2D_ERR_UNSUPPORTED;
  if (misaligned(qkv, 16) || misaligned(cos, 16) || misaligned(sin, 16) || misaligned(out, 16) || misaligned(q_weight, 16) ||
      misaligned(q_bias, 16) || misaligned(k_weight, 16) || misaligned(k_bias, 16))
    return M2D_ERR_MISALIGNED;
  AttnArgs a = {};
  a.qkv = qkv; a.cos = cos; a.sin = sin; a.qw = q_weight; a.qb = q_bias; a.kw = k_weight; a.kb = k_bias; a.out = out;
  a.L = L; a.heads = heads; a.wbf16 = weight_dtype == M2D_BF16; a.eps = eps; a.scale_log2e = scale * 1.44269504088896341f;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const unsigned blocks = (unsigned)((int64_t)B * heads);
  switch ((L + 15) / 16) {
    case 1: launch_attention<1>(a, blocks, st); break;
    case 2: launch_attention<2>(a, blocks, st); break;
    case 3: launch_attention<3>(a, blocks, st); break;
    case 4: launch_attention<4>(a, blocks, st); break;
    case 5: launch_attention<5>(a, blocks, st); break;
    case 6: launch_attention<6>(a, blocks, st); break;
    case 7: launch_attention<7>(a, blocks, st); break;
    case 8: launch_attention<8>(a, blocks, st); break;
    case 9: launch_attention<9>(a, blocks, st); break;
    case 10: launch_attention<10>(a, blocks, st); break;
    case 11: launch_attention<11>(a, blocks, st); break;
    case 12: launch_attention<12>(a, blocks, st); break;
    case 13: launch_attention<13>(a, blocks, st); break;
    case 14: launch_attention<14>(a, blocks, st); break;
    case 15: launch_attention<15>(a, blocks, st); break;
    default: launch_attention<16>(a, blocks, st); break;
  }
  return hipGetLastError() == hipSuccess ? M2D_OK : M2D_ERR_HIP;
}

static int run_linear(int64_t P, int K, int N, int weight_dtype, const void* x, const void* weight, const void* bias,
                      int pre_act, const void* pre_scale, const void* pre_bias, int post_act, const void* post_scale,
                      const void* post_bias, void* y, void* stream, const void* ln_w, const void* ln_b, float ln_eps) {
  if (!x || !weight || !y) return M2D_ERR_NULL_POINTER;
  const bool ln = pre_act == kActLayerNorm;
  if (ln && (!ln_w || !ln_b)) return M2D_ERR_NULL_POINTER;
  if ((pre_act == kActStarRelu && (!pre_scale || !pre_bias)) || (post_act == kActStarRelu && (!post_scale || !post_bias)))
    return M2D_ERR_NULL_POINTER;
  if (P < 1 || K < 1 || N < 1) return M2D_ERR_BAD_SHAPE;
  if (weight_dtype != M2D_F32 && weight_dtype != M2D_BF16) return M2D_ERR_UNSUPPORTED;
  if (pre_act < kActNone || pre_act > kActLayerNorm || post_act < kActNone || post_act > kActStarRelu) return M2D_ERR_UNSUPPORTED;
  if (K % 32 != 0 || K > 32 * kLinMaxKC || N % 16 != 0) return M2D_ERR_UNSUPPORTED;
  if (ln && K > 128) return M2D_ERR_UNSUPPORTED;      // the normalised rows live in registers next to the operands
  // Slices of the outputs, so that a workgroup's share of the weights leaves room for four workgroups on a
  // compute unit (each slice reads the rows of x again; they are the smaller side where N is large).
  int nsplit = 1;
  while (linear_lds_bytes(K, N / nsplit, ln) > 40 * 1024 && (N / nsplit) % 32 == 0 && N / nsplit > 64) nsplit *= 2;
  const int Ns = N / nsplit;
  if (linear_lds_bytes(K, Ns, ln) > kLinMaxLds) return M2D_ERR_UNSUPPORTED;
  if ((P + 63) / 64 >= ((int64_t)1 << 31)) return M2D_ERR_UNSUPPORTED;
  if (misaligned(x, 16) || misaligned(y, 16) || misaligned(weight, 16) || (bias && misaligned(bias, 4))) return M2D_ERR_MISALIGNED;
  if (ln && (misaligned(ln_w, 4) || misaligned(ln_b, 4))) return M2D_ERR_MISALIGNED;
  LinArgs a = {};
  a.ln_w = ln_w; a.ln_b = ln_b; a.ln_eps = ln_eps;
  a.x = x; a.w = weight; a.bias = bias; a.y = y; a.P = P; a.K = K; a.N = N; a.wbf16 = weight_dtype == M2D_BF16;
  a.pre = pre_act; a.post = post_act; a.pre_s = pre_scale; a.pre_b = pre_bias; a.post_s = post_scale; a.post_b = post_bias;
  a.ntiles = (int)((P + 63) / 64);
  a.nsplit = nsplit; a.Ns = Ns;
  const size_t lds = linear_lds_bytes(K, Ns, ln);
  if (lds > 64 * 1024 && !allow_big_lds()) return M2D_ERR_HIP;
  // persistent: the weights are loaded into LDS once per workgroup; as many workgroups as fit the device at once
  int per_cu = (int)(160 * 1024 / lds);
  if (per_cu > 8) per_cu = 8;
  int grid = 256 * per_cu / nsplit;     // workgroups per slice
  if (grid > a.ntiles) grid = a.ntiles;
  if (grid < 1) grid = 1;
  grid *= nsplit;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 g((unsigned)grid), t(kLinThreads);
  if (K <= 64) hipLaunchKernelGGL(m2d_linear_kernel<2>, g, t, lds, st, a);
  else if (K <= 128) hipLaunchKernelGGL(m2d_linear_kernel<4>, g, t, lds, st, a);
  else if (K <= 256) hipLaunchKernelGGL(m2d_linear_kernel<8>, g, t, lds, st, a);
  else hipLaunchKernelGGL(m2d_linear_kernel<16>, g, t, lds, st, a);
  return hipGetLastError() == hipSuccess ? M2D_OK : M2D_ERR_HIP;
}

int m2d_linear_fwd(int64_t P, int K, int N, int weight_dtype, const void* x, const void* weight, const void* bias,
                   int pre_act, const void* pre_scale, const void* pre_bias, int post_act, const void* post_scale,
                   const void* post_bias, void* y, void* stream) {
  if (pre_act == kActLayerNorm) return M2D_ERR_UNSUPPORTED;      // that one has an entry point of its own
  return run_linear(P, K, N, weight_dtype, x, weight, bias, pre_act, pre_scale, pre_bias, post_act, post_scale, post_bias, y, stream,
                    nullptr, nullptr, 0.f);
}

int m2d_layernorm_linear_fwd(int64_t P, int K, int N, int weight_dtype, const void* x, const void* ln_weight, const void* ln_bias,
                             float eps, const void* weight, const void* bias, int post_act, const void* post_scale,
                             const void* post_bias, void* y, void* stream) {
  return run_linear(P, K, N, weight_dtype, x, weight, bias, kActLayerNorm, nullptr, nullptr, post_act, post_scale, post_bias, y, stream,
                    ln_weight, ln_bias, eps);
}

}  // extern "C"

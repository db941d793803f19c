// Projections either side of the 2-D selective scan, for gfx950.
//
// The reference derives the scan's parameters from x with three library GEMMs and a softplus
// (proj_params, models/kernels/wavefront_cuda.py:63-95) and leaves their backward to autograd
// (wavefront_cuda.py:262-296).  The products are skinny -- the inner dimensions are d_model,
// dt_rank and 2*dt_rank + 3*d_state -- and the weight gradients reduce over every position of
// the batch, which general GEMM libraries handle poorly.  Here each pass is a few kernels that
// walk the (position, channel) arrays once, a tile of 64 positions at a time:
//
//   forward   z = x Wx^T ;  [rT | rL | B_T | B_L | C] = z ;  delta = softplus(r w^T + b)
//   backward  dpre = d_delta * (1 - exp(-delta))            (softplus'(pre) = 1 - exp(-softplus(pre)))
//             dz = [dpreT wT | dpreL wL | dB_T | dB_L | dC] ;  dx += dz Wx
//             dWx = dz^T x ;  dw = dpre^T r ;  db = sum dpre      (sums over all positions)
//
// Arithmetic is fp32 on the vector ALUs: a thread owns one position of the tile and multiplies
// it with weights that are uniform over the wave, so the weights arrive through scalar loads and
// cost no vector registers or LDS traffic.  The host packs the weights once per call into padded,
// transposed copies so that those loads are aligned runs of 16 floats with no edge cases.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "m2dscan.h"

namespace {

constexpr int kN = 16;        // d_state the scan is built for
constexpr int kTP = 64;       // positions per tile (one per lane)
constexpr int kKC = 64;       // channels per chunk of the inner dimension
constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;
constexpr int kXS = kKC + 1;  // row stride (floats) of a 64 x 64 tile in LDS, odd: lanes reading one column hit 64 banks
constexpr int kXS4 = kKC + 4; // the same for tiles read as float4
constexpr int kMaxR = 32;     // largest dt_rank
constexpr int kMaxRounds = 4; // 16-wide output chunks per wave

struct bf16_t { uint16_t v; };

__device__ __forceinline__ float ld(const float* p) { return *p; }
__device__ __forceinline__ float ld(const bf16_t* p) { return __uint_as_float((uint32_t)p->v << 16); }
// round to nearest even; the conversion is one instruction on gfx950 (v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16_pair(float lo, float hi) {   // one v_cvt_pk_bf16_f32
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
__device__ __forceinline__ void st(float* p, float v) { *p = v; }
__device__ __forceinline__ void st(bf16_t* p, float v) { p->v = f32_to_bf16_bits(v); }
// the value a tensor of type T would hold
__device__ __forceinline__ float as_stored(float v, const float*) { return v; }
__device__ __forceinline__ float as_stored(float v, const bf16_t*) { return __uint_as_float((uint32_t)f32_to_bf16_bits(v) << 16); }

// exp and log as the bare hardware instructions: the arguments below stay in ranges that
// need none of the library's scaling (results that underflow may flush to zero).
__device__ __forceinline__ float exp_neg(float v) { return __builtin_amdgcn_exp2f(v * 1.44269504088896341f); }   // v <= 0

// softplus with torch's defaults (beta 1; above the threshold of 20 the two agree in fp32):
// max(v,0) + log1p(t), t = exp(-|v|), with log1p(t) = log(u) + (t - (u-1)) for u = fl(1+t): the
// second term makes up for the rounding of 1+t when t is small.  (Exactly it would be divided by u;
// it is at most half an ulp of u, 6e-8, and u lies in [1, 2], so leaving the division out changes
// the result by less than 6e-8 t.)
__device__ __forceinline__ float softplus(float v) {
  const float t = exp_neg(-fabsf(v));
  const float u = 1.f + t;
  return fmaxf(v, 0.f) + __builtin_fmaf(__builtin_amdgcn_logf(u), 0.693147180559945309f, t - (u - 1.f));
}
// d softplus / d pre, from the softplus value: sigmoid(pre) = 1 - exp(-softplus(pre)).  Small
// arguments take the series, where 1 - exp(-d) would cancel.
__device__ __forceinline__ float softplus_slope(float d) {
  const float series = d * __builtin_fmaf(d, __builtin_fmaf(d, __builtin_fmaf(d, -1.f / 24.f, 1.f / 6.f), -0.5f), 1.f);
  return d < 0.0625f ? series : 1.f - exp_neg(-d);
}

// Where the scan kernels expect value n (0..47: B_T, B_L, C, 16 states each) inside a position's
// record of 48 floats: the four states n = 4q + m, q = 0..3, that the scan's backward folds together
// share a float4, in the order q = 0, 2, 1, 3 (the scan source calls this the fold order).
__device__ __forceinline__ int record_slot(int n48) {
  const int n = n48 & 15, q = n >> 2, m = n & 3;
  return (n48 & ~15) + 4 * m + (q == 1 ? 2 : (q == 2 ? 1 : q));
}

struct ProjArgs {
  // activations, (P, .) row-major, element type T
  const void *x, *r, *dT, *dL;           // x (P,E); r (P,2R) = low-rank inputs of the two dt projections; delta (P,E)
  const void *ddT, *ddL, *dBT, *dBL, *dC;
  int dpre_given;                        // ddT, ddL hold the gradients before the softplus already (dT, dL are not read)
  int sum_parts;                         // > 0: dBT points to that many fp32 records [P][dC | dBT | dBL][16] to add up (the scan's per-workgroup sums)
  void *r_out, *dT_out, *dL_out, *BT_out, *BL_out, *C_out, *dx;
  float* bc_packed;                      // (P,48) fp32 records for the scan kernels instead of BT_out, BL_out, C_out (or null)
  // packed weights, fp32, zero where padded
  const float *Wt;                       // [Epad][Opad]   Wx transposed
  const float *wTt, *wLt;                // [R][Epad]      dt weights transposed
  const float *bTp, *bLp;                // [Epad]
  const float *Wp;                       // [O][Epad]      Wx
  const float *wTp, *wLp;                // [Epad][Rpad]   dt weights
  // packed weights for the matrix-core kernels, bf16, zero where padded
  const uint16_t *Wb;                    // [Opad][Epad]   Wx
  const uint16_t *wTb, *wLb;             // [Epad][32]     dt weights
  const uint16_t *wTtb, *wLtb;           // [Rpad][Epad]   dt weights transposed
  const uint16_t *WxTb;                  // [Epad][Opad32] Wx transposed
  float* dz;                             // (P,O4) fp32, rows padded to a multiple of 4
  // the same for the matrix-core kernels, bf16
  uint16_t* dzt;                         // (P16, Opad)    dz, P16 = positions rounded up to 16
  uint16_t* dpt;                         // [2](P16, E)    dpreT, dpreL
  float* part;                           // per-workgroup sums of the weight gradients
  float *dWx, *dwT, *dbT, *dwL, *dbL;    // outputs of the reduction
  int64_t P;
  int E, R, O, O4, Epad, Opad, Opad32, Rpad;
  int ntiles, G, ne;
};

// Packed weights are read through the constant address space: they were written by an earlier
// launch, and a wave-uniform load from that space is a scalar load whatever the kernel stores.
typedef const __attribute__((address_space(4))) float* const_floats;
__device__ __forceinline__ const_floats as_const(const float* p) { return (const_floats)(uintptr_t)p; }

__device__ __forceinline__ int wave_id() { return __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)); }

// ------------------------------------------------------------------------------- weights
struct PackArgs {
  const float *Wx, *wT, *bT, *wL, *bL;
  float *Wt, *wTt, *wLt, *bTp, *bLp;     // forward set (or null)
  float *Wp, *wTp, *wLp;                 // backward set (or null)
  uint16_t *Wb, *wTb, *wLb;              // forward set of the matrix-core kernels (or null)
  uint16_t *wTtb, *wLtb, *WxTb;          // backward set of the matrix-core kernels (or null)
  int E, R, O, Epad, Opad, Opad32, Rpad;
  int round;                             // round every weight to bf16 first (the bf16 copies are rounded anyway)
};

// Padded copies of the weights.  One thread per element of the largest copy.
__global__ void m2d_proj_pack_kernel(const PackArgs k) {
  // a weight as the kernels are to see it
  auto w = [&](const float* p, int i) { return k.round ? as_stored(p[i], static_cast<const bf16_t*>(nullptr)) : p[i]; };
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (k.Wt) {
    if (i < k.Epad * k.Opad) {
      const int e = i / k.Opad, o = i - e * k.Opad;
      k.Wt[i] = (e < k.E && o < k.O) ? w(k.Wx, o * k.E + e) : 0.f;
    }
    if (i < k.R * k.Epad) {
      const int q = i / k.Epad, e = i - q * k.Epad;
      k.wTt[i] = e < k.E ? w(k.wT, e * k.R + q) : 0.f;
      k.wLt[i] = e < k.E ? w(k.wL, e * k.R + q) : 0.f;
    }
  }
  if (k.bTp && i < k.Epad) {
    k.bTp[i] = i < k.E ? w(k.bT, i) : 0.f;
    k.bLp[i] = i < k.E ? w(k.bL, i) : 0.f;
  }
  if (k.Wb) {
    if (i < k.Opad * k.Epad) {
      const int o = i / k.Epad, e = i - o * k.Epad;
      k.Wb[i] = (o < k.O && e < k.E) ? f32_to_bf16_bits(k.Wx[o * k.E + e]) : 0;
    }
    if (i < k.Epad * 32) {
      const int e = i >> 5, q = i & 31;
      const bool ok = e < k.E && q < k.R;
      k.wTb[i] = ok ? f32_to_bf16_bits(k.wT[e * k.R + q]) : 0;
      k.wLb[i] = ok ? f32_to_bf16_bits(k.wL[e * k.R + q]) : 0;
    }
  }
  if (k.WxTb) {
    if (i < k.Epad * k.Opad32) {
      const int e = i / k.Opad32, o = i - e * k.Opad32;
      k.WxTb[i] = (o < k.O && e < k.E) ? f32_to_bf16_bits(k.Wx[o * k.E + e]) : 0;
    }
    if (i < k.Rpad * k.Epad) {
      const int q = i / k.Epad, e = i - q * k.Epad;
      const bool ok = e < k.E && q < k.R;
      k.wTtb[i] = ok ? f32_to_bf16_bits(k.wT[e * k.R + q]) : 0;
      k.wLtb[i] = ok ? f32_to_bf16_bits(k.wL[e * k.R + q]) : 0;
    }
  }
  if (k.Wp) {
    if (i < k.O * k.Epad) {
      const int o = i / k.Epad, e = i - o * k.Epad;
      k.Wp[i] = e < k.E ? w(k.Wx, o * k.E + e) : 0.f;
    }
    if (i < k.Epad * k.Rpad) {
      const int e = i / k.Rpad, q = i - e * k.Rpad;
      const bool ok = e < k.E && q < k.R;
      k.wTp[i] = ok ? w(k.wT, e * k.R + q) : 0.f;
      k.wLp[i] = ok ? w(k.wL, e * k.R + q) : 0.f;
    }
  }
}

// ------------------------------------------------------------------------------- tiles
// A tile is 64 positions x 64 channels of a (P,E) array, 16 elements per thread.  The loads of a
// tile are issued back to back into registers and converted when they are consumed, so that a
// thread waits for memory once per tile and not once per row.
// VEC (E a multiple of the 16-byte vector): thread t holds, for l < NL, the EPL elements from
//   column (ci % CPR) * EPL of row ci / CPR, ci = l * 256 + t.  Otherwise element i = l * 256 + t,
//   row i / 64, column i % 64.
template <typename T, bool VEC>
struct Tile {
  static constexpr int EPL = VEC ? 16 / (int)sizeof(T) : 1;
  static constexpr int NL = 16 / EPL;
  static constexpr int CPR = kKC / EPL;
  struct Regs { uint4 q[VEC ? NL : 1]; float v[VEC ? 1 : 16]; };

  static __device__ __forceinline__ void pos(int t, int l, int& row, int& col) {
    const int ci = l * kThreads + t;
    row = ci / CPR;
    col = (ci % CPR) * EPL;
  }
  static __device__ __forceinline__ void load(Regs& r, const T* base, int64_t p0, int64_t P, int E, int e0, int t) {
#pragma unroll
    for (int l = 0; l < NL; ++l) {
      int row, col;
      pos(t, l, row, col);
      const int64_t p = p0 + row;
      const bool ok = p < P && e0 + col < E;
      if constexpr (VEC) r.q[l] = ok ? *reinterpret_cast<const uint4*>(base + p * E + e0 + col) : make_uint4(0, 0, 0, 0);
      else r.v[l] = ok ? ld(base + p * E + e0 + col) : 0.f;
    }
  }
  // element j < EPL of load l
  static __device__ __forceinline__ float get(const Regs& r, int l, int j) {
    if constexpr (!VEC) return r.v[l];
    else {
      const uint32_t w[4] = {r.q[l].x, r.q[l].y, r.q[l].z, r.q[l].w};
      if constexpr (sizeof(T) == 4) return __uint_as_float(w[j]);
      else return __uint_as_float((j & 1) ? (w[j >> 1] & 0xffff0000u) : (w[j >> 1] << 16));
    }
  }
  // v(l, j) for every element -> tile[row * stride + col]
  template <typename F>
  static __device__ __forceinline__ void to_lds(float* tile, int stride, int t, F value) {
#pragma unroll
    for (int l = 0; l < NL; ++l) {
      int row, col;
      pos(t, l, row, col);
#pragma unroll
      for (int j = 0; j < EPL; ++j) tile[row * stride + col + j] = value(l, j);
    }
  }
  // tile[row * stride + col] (+ what `plus` holds) -> global, rows and channels inside the array only
  static __device__ __forceinline__ void store(const float* tile, int stride, T* base, int64_t p0, int64_t P, int E, int e0,
                                               int t, const Regs* plus) {
#pragma unroll
    for (int l = 0; l < NL; ++l) {
      int row, col;
      pos(t, l, row, col);
      const int64_t p = p0 + row;
      if (!(p < P && e0 + col < E)) continue;
      float v[EPL];
#pragma unroll
      for (int j = 0; j < EPL; ++j) v[j] = tile[row * stride + col + j] + (plus ? get(*plus, l, j) : 0.f);
      T* dst = base + p * E + e0 + col;
      if constexpr (!VEC) st(dst, v[0]);
      else if constexpr (sizeof(T) == 4) *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
      else {
        uint32_t w[4];
#pragma unroll
        for (int h = 0; h < 4; ++h) w[h] = pack_bf16_pair(v[2 * h], v[2 * h + 1]);
        *reinterpret_cast<uint4*>(dst) = make_uint4(w[0], w[1], w[2], w[3]);
      }
    }
  }
};

// acc[j] += sum_e tile[lane][e] * w[e * stride + j], e < 64, j < 16; w is uniform over the wave
__device__ __forceinline__ void row_times_weights(const float* tile_row, const_floats w, int stride, float (&acc)[16]) {
#pragma unroll 4
  for (int e = 0; e < kKC; ++e) {
    const float v = tile_row[e];
    const_floats we = w + e * stride;
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[j] = __builtin_fmaf(v, we[j], acc[j]);
  }
}

// ------------------------------------------------------------------------------- forward
// One workgroup per tile of 64 positions.  LDS: xs[64][65] (a chunk of x, later the deltaT tile),
// zs[64][O+1] (z), outL[64][65] (the deltaL tile).
template <typename T, bool VEC>
__global__ __launch_bounds__(kThreads) void m2d_proj_fwd_kernel(const ProjArgs a) {
  using TL = Tile<T, VEC>;
  extern __shared__ float smem[];
  float* xs = smem;
  float* zs = smem + kTP * kXS;
  float* outL = zs + kTP * (a.O + 1);
  float* outT = xs;
  const int zst = a.O + 1;
  const int wave = wave_id(), lane = threadIdx.x & 63, tid = threadIdx.x;
  const int64_t p0 = (int64_t)blockIdx.x * kTP;
  const T* x = static_cast<const T*>(a.x);
  const int nOC = a.Opad / 16, nkc = a.Epad / kKC;

  float acc[kMaxRounds][16];
#pragma unroll
  for (int rd = 0; rd < kMaxRounds; ++rd)
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[rd][j] = 0.f;

  typename TL::Regs xr;
  TL::load(xr, x, p0, a.P, a.E, 0, tid);
  for (int kc = 0; kc < nkc; ++kc) {
    TL::to_lds(xs, kXS, tid, [&](int l, int j) { return TL::get(xr, l, j); });
    __syncthreads();
    if (kc + 1 < nkc) TL::load(xr, x, p0, a.P, a.E, (kc + 1) * kKC, tid);   // under way during the products
#pragma unroll
    for (int rd = 0; rd < kMaxRounds; ++rd) {
      const int oc = wave + kWaves * rd;
      if (oc < nOC) row_times_weights(xs + lane * kXS, as_const(a.Wt) + (int64_t)kc * kKC * a.Opad + oc * 16, a.Opad, acc[rd]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int rd = 0; rd < kMaxRounds; ++rd) {
    const int oc = wave + kWaves * rd;
    if (oc < nOC) {
#pragma unroll
      for (int j = 0; j < 16; ++j)
        if (oc * 16 + j < a.O) zs[lane * zst + oc * 16 + j] = acc[rd][j];
    }
  }
  __syncthreads();

  // ---- low-rank inputs and B_T, B_L, C: a row of the tile per wave at a time
  const int R = a.R, R2 = 2 * a.R;
  T* r_out = static_cast<T*>(a.r_out);
  for (int c = wave; c < kTP; c += kWaves) {
    const int64_t p = p0 + c;
    if (p >= a.P) break;   // uniform
    const float* z = zs + c * zst;
    for (int q = lane; q < R2; q += 64) st(r_out + p * R2 + q, z[q]);
    if (lane < 3 * kN) {
      if (a.bc_packed) {
        a.bc_packed[p * (3 * kN) + record_slot(lane)] = as_stored(z[R2 + lane], r_out);
      } else {
        T* out = static_cast<T*>(lane < kN ? a.BT_out : (lane < 2 * kN ? a.BL_out : a.C_out));
        st(out + p * kN + (lane & (kN - 1)), z[R2 + lane]);
      }
    }
  }

  // ---- delta = softplus(r w^T + b), 64 channels at a time: a thread works out 16 channels of
  // its position with wave-uniform weights, the tile goes out row-wise through LDS
  const float* zrow = zs + lane * zst;
  for (int eg = 0; eg < nkc; ++eg) {
    const int e0 = eg * kKC + wave * 16;
    float sT[16], sL[16];
    const_floats bt = as_const(a.bTp) + e0;
    const_floats bl = as_const(a.bLp) + e0;
#pragma unroll
    for (int j = 0; j < 16; ++j) { sT[j] = bt[j]; sL[j] = bl[j]; }
    for (int q = 0; q < R; ++q) {
      // the dt projections see the low-rank inputs as the tensor holds them
      const float zT = as_stored(zrow[q], r_out), zL = as_stored(zrow[R + q], r_out);
      const_floats wt = as_const(a.wTt) + q * a.Epad + e0;
      const_floats wl = as_const(a.wLt) + q * a.Epad + e0;
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        sT[j] = __builtin_fmaf(zT, wt[j], sT[j]);
        sL[j] = __builtin_fmaf(zL, wl[j], sL[j]);
      }
    }
    if (eg > 0) __syncthreads();   // the tiles of the previous group have gone out
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      outT[lane * kXS + wave * 16 + j] = softplus(sT[j]);
      outL[lane * kXS + wave * 16 + j] = softplus(sL[j]);
    }
    __syncthreads();
    TL::store(outT, kXS, static_cast<T*>(a.dT_out), p0, a.P, a.E, eg * kKC, tid, nullptr);
    TL::store(outL, kXS, static_cast<T*>(a.dL_out), p0, a.P, a.E, eg * kKC, tid, nullptr);
  }
}

// ------------------------------------------------------------------------------- backward, data
// One workgroup per tile.  LDS: dps[2][64][65] (chunks of dpreT, dpreL; reused for the dx tile),
// dzs[64][O+1].  Writes dz for the weight-gradient kernel and adds dz Wx to dx.
template <typename T, bool VEC>
__global__ __launch_bounds__(kThreads) void m2d_proj_bwd_data_kernel(const ProjArgs a) {
  using TL = Tile<T, VEC>;
  extern __shared__ float smem[];
  float* dps = smem;
  float* dzs = smem + 2 * kTP * kXS;
  const int zst = a.O + 1;
  const int wave = wave_id(), lane = threadIdx.x & 63, tid = threadIdx.x;
  const int64_t p0 = (int64_t)blockIdx.x * kTP;
  const int R = a.R, R2 = 2 * a.R;
  const int nRC = a.Rpad / 16;   // 16-wide chunks of one dt weight; 2*nRC chunks in all (T then L)
  const int nkc = a.Epad / kKC;
  const T* dT = static_cast<const T*>(a.dT);
  const T* dL = static_cast<const T*>(a.dL);
  const T* ddT = static_cast<const T*>(a.ddT);
  const T* ddL = static_cast<const T*>(a.ddL);
  const bool given = a.dpre_given != 0;   // (uniform) ddT, ddL are dpre already
  const int64_t Pv = given ? 0 : a.P;     // rows of deltaT, deltaL to read: none then

  // dB_T, dB_L, dC of the tile: 64 x 16 contiguous elements each, 4 per thread
  float bc[3][4];
#pragma unroll
  for (int w = 0; w < 3; ++w) {
    const T* src = static_cast<const T*>(w == 0 ? a.dBT : (w == 1 ? a.dBL : a.dC));
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int i = k * kThreads + tid;
      bc[w][k] = p0 + (i >> 4) < a.P ? ld(src + p0 * kN + i) : 0.f;
    }
  }

  float acc[kMaxRounds][16];
#pragma unroll
  for (int rd = 0; rd < kMaxRounds; ++rd)
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[rd][j] = 0.f;

  for (int kc = 0; kc < nkc; ++kc) {
    typename TL::Regs gT, vT, gL, vL;
    TL::load(gT, ddT, p0, a.P, a.E, kc * kKC, tid);
    TL::load(vT, dT, p0, Pv, a.E, kc * kKC, tid);
    TL::load(gL, ddL, p0, a.P, a.E, kc * kKC, tid);
    TL::load(vL, dL, p0, Pv, a.E, kc * kKC, tid);
    TL::to_lds(dps, kXS, tid, [&](int l, int j) { return TL::get(gT, l, j) * (given ? 1.f : softplus_slope(TL::get(vT, l, j))); });
    TL::to_lds(dps + kTP * kXS, kXS, tid, [&](int l, int j) { return TL::get(gL, l, j) * (given ? 1.f : softplus_slope(TL::get(vL, l, j))); });
    __syncthreads();
#pragma unroll
    for (int rd = 0; rd < kMaxRounds; ++rd) {
      const int ci = wave + kWaves * rd;
      if (ci < 2 * nRC) {
        const bool isL = ci >= nRC;
        const int qc = isL ? ci - nRC : ci;
        row_times_weights(dps + (isL ? kTP * kXS : 0) + lane * kXS,
                          as_const(isL ? a.wLp : a.wTp) + (int64_t)kc * kKC * a.Rpad + qc * 16, a.Rpad, acc[rd]);
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int rd = 0; rd < kMaxRounds; ++rd) {
    const int ci = wave + kWaves * rd;
    if (ci < 2 * nRC) {
      const bool isL = ci >= nRC;
      const int qc = isL ? ci - nRC : ci;
#pragma unroll
      for (int j = 0; j < 16; ++j)
        if (qc * 16 + j < R) dzs[lane * zst + (isL ? R : 0) + qc * 16 + j] = acc[rd][j];
    }
  }
#pragma unroll
  for (int w = 0; w < 3; ++w)
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int i = k * kThreads + tid;
      dzs[(i >> 4) * zst + R2 + w * kN + (i & 15)] = bc[w][k];
    }
  __syncthreads();

  for (int c = wave; c < kTP; c += kWaves) {
    const int64_t p = p0 + c;
    if (p >= a.P) break;   // uniform
    for (int o = lane; o < a.O4; o += 64) a.dz[p * a.O4 + o] = o < a.O ? dzs[c * zst + o] : 0.f;
  }

  // ---- dx += dz Wx, 64 channels at a time (16 per wave), through LDS for row-wise stores
  T* dx = static_cast<T*>(a.dx);
  float* outs = dps;
  for (int eg = 0; eg < nkc; ++eg) {
    typename TL::Regs old;
    TL::load(old, dx, p0, a.P, a.E, eg * kKC, tid);
    float s[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) s[j] = 0.f;
    const_floats w = as_const(a.Wp) + eg * kKC + wave * 16;
    const float* zrow = dzs + lane * zst;
#pragma unroll 2
    for (int o = 0; o < a.O; ++o) {
      const float v = zrow[o];
      const_floats wo = w + (int64_t)o * a.Epad;
#pragma unroll
      for (int j = 0; j < 16; ++j) s[j] = __builtin_fmaf(v, wo[j], s[j]);
    }
    if (eg > 0) __syncthreads();   // the previous tile has gone out
#pragma unroll
    for (int j = 0; j < 16; ++j) outs[lane * kXS + wave * 16 + j] = s[j];
    __syncthreads();
    TL::store(outs, kXS, dx, p0, a.P, a.E, eg * kKC, tid, &old);
  }
}

// ------------------------------------------------------------------------------- matrix cores
// bf16 tensors whose rows start on 16-byte boundaries take the products through
// v_mfma_f32_16x16x32_bf16.  A wave owns 16 positions and needs nothing from the other waves of
// its workgroup.  Operand layout of the instruction (lane l, m = n = l & 15, kb = l >> 4):
//   A[m][8 kb + j], B[8 kb + j][n] (j < 8, one 16-byte register set each);  D[4 kb + i][n], i < 4.
// With positions as rows of A, the 8 values a lane needs are 8 consecutive channels of one
// position: one 16-byte load straight from the (P,E) array.  The weights are packed so that the
// same holds for B.
#ifndef M2D_PROJ_OCC
#define M2D_PROJ_OCC 5
#endif
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
constexpr int kMaxNT = (2 * kMaxR + 3 * kN + 15) / 16;   // 16-wide tiles of the 2R+48 outputs
constexpr int kLowStride = 40;   // bf16 per row of the low-rank scratch: 32 + 8, rows 16-byte aligned and spread over the banks

__device__ __forceinline__ f32x4 mfma16(uint4 a, uint4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}
// written out at every use: as a named constant the register allocator has kept it in scratch memory
__device__ __forceinline__ uint4 zero16() { return make_uint4(0u, 0u, 0u, 0u); }
__device__ __forceinline__ uint4 load16(const void* p) { return *reinterpret_cast<const uint4*>(p); }
__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2){lo, hi}, bf16x2));
}

// Results leave the accumulators (4 positions x 1 channel per lane and tile) through a per-wave
// LDS block of 16 positions x 64 channels, so that memory sees 16-byte pieces of rows.
constexpr int kStageStride = 72;   // floats per row: 64 + 8, rows 16-byte aligned (also holds 2 x [16][72] bf16)
__device__ __forceinline__ void wave_sync_lds() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
__device__ __forceinline__ void stage_put(float* stage, int nt, int mn, int kb, f32x4 v) {
#pragma unroll
  for (int i = 0; i < 4; ++i) stage[(4 * kb + i) * kStageStride + 16 * nt + mn] = v[i];
}
// f(position, first channel, 8 values) for the lane's two pieces of the block
template <typename F>
__device__ __forceinline__ void stage_rows(const float* stage, int l, F f) {
#pragma unroll
  for (int k = 0; k < 2; ++k) {
    const int piece = l + 64 * k, c = piece >> 3, c8 = 8 * (piece & 7);
    const float4 lo = *reinterpret_cast<const float4*>(stage + c * kStageStride + c8);
    const float4 hi = *reinterpret_cast<const float4*>(stage + c * kStageStride + c8 + 4);
    const float v[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    f(c, c8, v);
  }
}
__device__ __forceinline__ uint4 pack8(const float (&v)[8]) {
  return make_uint4(pack2(v[0], v[1]), pack2(v[2], v[3]), pack2(v[4], v[5]), pack2(v[6], v[7]));
}

// Forward.  LDS: per wave two [16][40] bf16 blocks (low-rank inputs of the T and L projection)
// and the [16][68] fp32 block the delta tiles leave through.
__global__ __launch_bounds__(kThreads, M2D_PROJ_OCC) void m2d_proj_fwd_mfma_kernel(const ProjArgs a) {
  extern __shared__ float smem[];
  const int wave = wave_id(), l = threadIdx.x & 63, mn = l & 15, kb = l >> 4;
  float* stage = smem + wave * (16 * kStageStride + 16 * kLowStride);   // [16][68] floats, then 2 x [16][40] bf16
  uint16_t* lowT = reinterpret_cast<uint16_t*>(stage + 16 * kStageStride);
  uint16_t* lowL = lowT + 16 * kLowStride;
  // columns past the rank meet zero weights; they only have to be finite
  for (int i = l; i < 16 * kLowStride; i += 64) reinterpret_cast<uint32_t*>(lowT)[i] = 0u;
  const int64_t p0 = (int64_t)blockIdx.x * kTP + wave * 16;
  const bf16_t* x = static_cast<const bf16_t*>(a.x);
  const int64_t pm = p0 + mn;
  const int NT = a.Opad / 16, R = a.R, R2 = 2 * a.R;

  f32x4 acc[kMaxNT];
#pragma unroll
  for (int nt = 0; nt < kMaxNT; ++nt) acc[nt] = (f32x4){0.f, 0.f, 0.f, 0.f};
  for (int e = 8 * kb; e < a.Epad; e += 32) {
    const uint4 A = (pm < a.P && e < a.E) ? load16(x + pm * a.E + e) : make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int nt = 0; nt < kMaxNT; ++nt)
      if (nt < NT) acc[nt] = mfma16(A, load16(a.Wb + (16 * nt + mn) * a.Epad + e), acc[nt]);
  }

  // z[position 4 kb + i][output 16 nt + mn]: low-rank inputs, B_T, B_L, C.  Addresses are a
  // wave-uniform base (the wave's first position) plus a 32-bit element offset.
  const int rows = (int)(a.P - p0 < 16 ? a.P - p0 : 16);   // positions of the wave inside the array (may be <= 0)
  bf16_t* r_out = static_cast<bf16_t*>(a.r_out) + p0 * R2;
  bf16_t* bt_out = static_cast<bf16_t*>(a.BT_out) + p0 * kN;
  bf16_t* bl_out = static_cast<bf16_t*>(a.BL_out) + p0 * kN;
  bf16_t* c_out = static_cast<bf16_t*>(a.C_out) + p0 * kN;
#pragma unroll
  for (int nt = 0; nt < kMaxNT; ++nt) {
    if (nt >= NT) break;
    const int o = 16 * nt + mn;
    const int oo = o - R2;
    bf16_t* bc = (oo < kN ? bt_out : (oo < 2 * kN ? bl_out : c_out)) + (oo & (kN - 1));
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = 4 * kb + i;
      const uint16_t h = f32_to_bf16_bits(acc[nt][i]);
      if (o < R) lowT[c * kLowStride + o] = h;
      else if (o < R2) lowL[c * kLowStride + o - R] = h;
      if (c < rows) {
        if (o < R2) r_out[(uint32_t)(c * R2 + o)].v = h;
        else if (o < a.O) {
          if (a.bc_packed) a.bc_packed[(p0 + c) * (3 * kN) + record_slot(oo)] = bf16_lo(h);
          else bc[(uint32_t)(c * kN)].v = h;
        }
      }
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

  // delta = softplus(low w^T + b): the rank is the inner dimension (one step of 32)
  const uint4 AT = load16(lowT + mn * kLowStride + 8 * kb), AL = load16(lowL + mn * kLowStride + 8 * kb);
  bf16_t* dT_out = static_cast<bf16_t*>(a.dT_out) + p0 * a.E;
  bf16_t* dL_out = static_cast<bf16_t*>(a.dL_out) + p0 * a.E;
  for (int e0 = 0; e0 < a.Epad; e0 += kKC) {
    f32x4 sT[4], sL[4];
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
      const int e = e0 + 16 * nt + mn;
      const float bT = a.bTp[e], bL = a.bLp[e];
      sT[nt] = mfma16(AT, load16(a.wTb + e * 32 + 8 * kb), (f32x4){bT, bT, bT, bT});
      sL[nt] = mfma16(AL, load16(a.wLb + e * 32 + 8 * kb), (f32x4){bL, bL, bL, bL});
    }
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) {
        const f32x4 v = h ? sL[nt] : sT[nt];
        stage_put(stage, nt, mn, kb, (f32x4){softplus(v[0]), softplus(v[1]), softplus(v[2]), softplus(v[3])});
      }
      wave_sync_lds();
      bf16_t* out = h ? dL_out : dT_out;
      stage_rows(stage, l, [&](int c, int c8, const float (&v)[8]) {
        if (c < rows && e0 + c8 < a.E) *reinterpret_cast<uint4*>(out + (uint32_t)(c * a.E + e0 + c8)) = pack8(v);
      });
      wave_sync_lds();
    }
  }
}

// Backward, data.  LDS: per wave one [16][Opad32 + 8] bf16 block (the rows of dz) and the [16][68]
// fp32 block the dx tiles leave through.  dz and dpre are also written out as bf16 arrays for the
// weight-gradient kernel.
__global__ __launch_bounds__(kThreads, M2D_PROJ_OCC) void m2d_proj_bwd_data_mfma_kernel(const ProjArgs a) {
  extern __shared__ float smem[];
  const int wave = wave_id(), l = threadIdx.x & 63, mn = l & 15, kb = l >> 4;
  const int zst = a.Opad32 + 8;
  float* stage = smem + wave * (16 * kStageStride + 16 * zst / 2);   // [16][68] floats, then [16][zst] bf16
  uint16_t* zs = reinterpret_cast<uint16_t*>(stage + 16 * kStageStride);
  for (int i = l; i < 16 * zst / 2; i += 64) reinterpret_cast<uint32_t*>(zs)[i] = 0u;   // padding columns: zero
  const int64_t p0 = (int64_t)blockIdx.x * kTP + wave * 16;
  const int rows = (int)(a.P - p0 < 16 ? a.P - p0 : 16);   // positions of the wave inside the array (may be <= 0)
  const int R = a.R, R2 = 2 * a.R, NQ = a.Rpad / 16;
  // wave-uniform bases (the wave's first position); lanes add 32-bit element offsets
  const bf16_t* dT = static_cast<const bf16_t*>(a.dT) + p0 * a.E;
  const bf16_t* dL = static_cast<const bf16_t*>(a.dL) + p0 * a.E;
  const bf16_t* ddT = static_cast<const bf16_t*>(a.ddT) + p0 * a.E;
  const bf16_t* ddL = static_cast<const bf16_t*>(a.ddL) + p0 * a.E;
  bf16_t* dx = static_cast<bf16_t*>(a.dx) + p0 * a.E;
  // rows past the end of the arrays (up to the next multiple of 16) are written too, as zeros
  uint16_t* dzt = a.dzt + p0 * a.Opad;
  uint16_t* dptT = a.dpt + p0 * a.E;
  uint16_t* dptL = dptT + (int64_t)a.ntiles * kTP * a.E;
  const uint4 z4 = make_uint4(0, 0, 0, 0);
  const bool given = a.dpre_given != 0;   // (uniform) ddT, ddL are dpre already: nothing to derive or to write out

  // Memory latency is covered by the other waves of the compute unit (registers are kept low
  // for that), not by fetching ahead.
  // dB_T, dB_L, dC: lane l holds 4 values of position l >> 2
  const int cb = l >> 2, n0 = 4 * (l & 3);
  uint2 bc[3];
  if (a.sum_parts > 0) {   // (uniform) the scan's per-workgroup channel sums, added up here in their order and rounded once
    const float* rec = static_cast<const float*>(a.dBT) + (p0 + cb) * (3 * kN) + n0;
#pragma unroll
    for (int w = 0; w < 3; ++w) {
      const int v = w == 0 ? 1 : (w == 1 ? 2 : 0);   // the records hold dC, dBT, dBL in this order
      float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
      if (cb < rows) {
        sum = *reinterpret_cast<const float4*>(rec + v * kN);
        for (int g = 1; g < a.sum_parts; ++g) {
          const float4 o = *reinterpret_cast<const float4*>(rec + (int64_t)g * a.P * (3 * kN) + v * kN);
          sum.x += o.x; sum.y += o.y; sum.z += o.z; sum.w += o.w;
        }
      }
      bc[w] = make_uint2(pack2(sum.x, sum.y), pack2(sum.z, sum.w));
    }
  } else {
#pragma unroll
    for (int w = 0; w < 3; ++w) {
      const bf16_t* src = static_cast<const bf16_t*>(w == 0 ? a.dBT : (w == 1 ? a.dBL : a.dC)) + p0 * kN;
      bc[w] = cb < rows ? *reinterpret_cast<const uint2*>(src + (uint32_t)(cb * kN + n0)) : make_uint2(0, 0);
    }
  }

  // dz[., rank] = dpre w, channels as the inner dimension
  f32x4 accT[2], accL[2];
#pragma unroll
  for (int nq = 0; nq < 2; ++nq) { accT[nq] = (f32x4){0.f, 0.f, 0.f, 0.f}; accL[nq] = accT[nq]; }
  auto dpre = [](uint4 g, uint4 v) {
    const uint32_t gw[4] = {g.x, g.y, g.z, g.w}, vw[4] = {v.x, v.y, v.z, v.w};
    uint32_t r[4];
#pragma unroll
    for (int h = 0; h < 4; ++h)
      r[h] = pack2(bf16_lo(gw[h]) * softplus_slope(bf16_lo(vw[h])), bf16_hi(gw[h]) * softplus_slope(bf16_hi(vw[h])));
    return make_uint4(r[0], r[1], r[2], r[3]);
  };
  for (int e = 8 * kb; e < a.Epad; e += 32) {
    const bool ok = mn < rows && e < a.E;
    const uint32_t off = (uint32_t)(mn * a.E + e);
    uint4 AT = ok ? load16(ddT + off) : z4, AL = ok ? load16(ddL + off) : z4;
    if (!given) {
      AT = dpre(AT, ok ? load16(dT + off) : z4);
      AL = dpre(AL, ok ? load16(dL + off) : z4);
    }
#pragma unroll
    for (int nq = 0; nq < 2; ++nq)
      if (nq < NQ) {
        accT[nq] = mfma16(AT, load16(a.wTtb + (16 * nq + mn) * a.Epad + e), accT[nq]);
        accL[nq] = mfma16(AL, load16(a.wLtb + (16 * nq + mn) * a.Epad + e), accL[nq]);
      }
    if (given) continue;   // the weight-gradient kernel reads the caller's arrays
    // dpre leaves through LDS, 64 channels at a time, so that memory sees whole 128-byte rows
    uint16_t* pst = reinterpret_cast<uint16_t*>(stage);
    *reinterpret_cast<uint4*>(pst + mn * kStageStride + (e & 63)) = AT;
    *reinterpret_cast<uint4*>(pst + (16 + mn) * kStageStride + (e & 63)) = AL;
    if ((e & 32) != 0) {   // uniform: second half of a group of 64
      const int e0 = e & ~63;
      wave_sync_lds();
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        const int piece = l + 64 * k, c = piece >> 3, c8 = 8 * (piece & 7);
        if (e0 + c8 < a.E) {
          *reinterpret_cast<uint4*>(dptT + (uint32_t)(c * a.E + e0 + c8)) = load16(pst + c * kStageStride + c8);
          *reinterpret_cast<uint4*>(dptL + (uint32_t)(c * a.E + e0 + c8)) = load16(pst + (16 + c) * kStageStride + c8);
        }
      }
      wave_sync_lds();
    }
  }
  // rows of dz to LDS as bf16: operand of the next product, and source of the copy in memory
#pragma unroll
  for (int nq = 0; nq < 2; ++nq) {
    const int q = 16 * nq + mn;
    if (nq < NQ && q < R) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = 4 * kb + i;
        zs[c * zst + q] = f32_to_bf16_bits(accT[nq][i]);
        zs[c * zst + R + q] = f32_to_bf16_bits(accL[nq][i]);
      }
    }
  }
#pragma unroll
  for (int w = 0; w < 3; ++w) {
    uint32_t* dst = reinterpret_cast<uint32_t*>(zs + cb * zst + R2 + w * kN + n0);   // even offsets: 4-byte aligned
    dst[0] = bc[w].x;
    dst[1] = bc[w].y;
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  {
    const int per_row = a.Opad / 8;   // 16-byte pieces of a row
    for (int i = l; i < 16 * per_row; i += 64) {
      const int c = i / per_row, o8 = i - c * per_row;
      *reinterpret_cast<uint4*>(dzt + (uint32_t)(c * a.Opad + 8 * o8)) = load16(zs + c * zst + 8 * o8);
    }
  }

  // dx += dz Wx, outputs as the inner dimension
  constexpr int kMaxKS = (2 * kMaxR + 3 * kN + 31) / 32;
  uint4 A2[kMaxKS];
#pragma unroll
  for (int ks = 0; ks < kMaxKS; ++ks)
    A2[ks] = 32 * ks < a.Opad32 ? load16(zs + mn * zst + 32 * ks + 8 * kb) : z4;
  for (int e0 = 0; e0 < a.Epad; e0 += kKC) {
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
      const int e = e0 + 16 * nt + mn;
      f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < kMaxKS; ++ks)
        if (32 * ks < a.Opad32) s = mfma16(A2[ks], load16(a.WxTb + e * a.Opad32 + 32 * ks + 8 * kb), s);
      stage_put(stage, nt, mn, kb, s);
    }
    wave_sync_lds();
    stage_rows(stage, l, [&](int c, int c8, const float (&v)[8]) {
      if (c < rows && e0 + c8 < a.E) {
        bf16_t* at = dx + (uint32_t)(c * a.E + e0 + c8);
        const uint4 was = load16(at);
        const uint32_t w[4] = {was.x, was.y, was.z, was.w};
        float sum[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) { sum[2 * j] = bf16_lo(w[j]) + v[2 * j]; sum[2 * j + 1] = bf16_hi(w[j]) + v[2 * j + 1]; }
        *reinterpret_cast<uint4*>(at) = pack8(sum);
      }
    });
    wave_sync_lds();
  }
}

// Backward, weights, on the matrix cores.  Positions are the inner dimension of all three sums,
//   dWx[o][e] = sum_p dz[p][o] x[p][e],  dw[e][q] = sum_p dpre[p][e] r[p][q],  db[e] = sum_p dpre[p][e] * 1,
// so every operand is wanted position-last while the arrays are position-first.  A tile of 64
// positions is turned in LDS: a lane loads 16 bytes of one position's row and writes its 8 values
// into 8 rows of the position-last block (lanes = consecutive positions: no bank conflicts).
// LDS: xT[64][72], pT[2][64][72], zT[Opad][72], rT[2][16 NQ1][72] with a row of ones after the
// R rows of r (its column of the product is db).  Grid, parts and the prefetch of the next tile
// are those of the vector-ALU kernel.
constexpr int kPosStride = 72;   // bf16 per row of a position-last block: 64 + 8, rows 16-byte aligned
constexpr int kMaxNQ1 = (kMaxR + 1 + 15) / 16;
constexpr int kMaxZP = (kMaxNT * 2 + kWaves - 1) / kWaves;   // 16-byte pieces of a dz row per wave

__global__ __launch_bounds__(kThreads) void m2d_proj_bwd_weights_mfma_kernel(const ProjArgs a) {
  extern __shared__ float smem[];
  const int wave = wave_id(), l = threadIdx.x & 63, mn = l & 15, kb = l >> 4, tid = threadIdx.x;
  const int ey = blockIdx.y;
  const int R = a.R, R2 = 2 * a.R;
  const int NQ1 = (R + 1 + 15) / 16, MT = a.Opad / 16, ZP = a.Opad / 8;
  uint16_t* xT = reinterpret_cast<uint16_t*>(smem);
  uint16_t* pT = xT + kKC * kPosStride;
  uint16_t* zT = pT + 2 * kKC * kPosStride;
  uint16_t* rT = zT + a.Opad * kPosStride;
  const int rblk = 16 * NQ1 * kPosStride;   // one tensor's block of rT
  for (int i = tid; i < rblk; i += kThreads) reinterpret_cast<uint32_t*>(rT)[i] = 0u;   // both blocks (2 * rblk / 2 words)
  __syncthreads();
  if (tid < 2 * kTP) rT[(tid >> 6) * rblk + R * kPosStride + (tid & 63)] = 0x3F80;   // 1.0
  const bf16_t* x = static_cast<const bf16_t*>(a.x);
  const bf16_t* rr = static_cast<const bf16_t*>(a.r);
  // dpre: the copy the data kernel wrote for whole tiles, or the caller's arrays (P rows)
  const bool given = a.dpre_given != 0;
  const uint16_t* dptT = given ? static_cast<const uint16_t*>(a.ddT) : a.dpt;
  const uint16_t* dptL = given ? static_cast<const uint16_t*>(a.ddL) : a.dpt + (int64_t)a.ntiles * kTP * a.E;

  // this thread's part of the r tile (64 x 2R values, contiguous): up to two 16-byte pieces
  int rp[2], rq[2];
#pragma unroll
  for (int k = 0; k < 2; ++k) {
    const int first = 8 * (k * kThreads + tid);
    rp[k] = first / R2;
    rq[k] = first - rp[k] * R2;
  }
  const int nr = kTP * R2;   // values in the r tile

  f32x4 aw[2][4], ar[2][kMaxNQ1];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) aw[h][nt] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int nq = 0; nq < kMaxNQ1; ++nq) ar[h][nq] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }

  uint4 xr[2], pr[2][2], zr[kMaxZP], rv[2];
  auto fetch = [&](int tile) {
    const int64_t p0 = (int64_t)tile * kTP;
    const int64_t left = a.P - p0;   // positions of the tile inside the array, if fewer than 64
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const int e = ey * kKC + 8 * (2 * wave + k);
      const bool ok = e < a.E;
      xr[k] = (l < left && ok) ? load16(x + (p0 + l) * a.E + e) : zero16();
      // dz and the data kernel's dpre are written for whole tiles (zeros past the end of the arrays)
      const bool pok = ok && (!given || l < left);
      pr[0][k] = pok ? load16(dptT + (p0 + l) * a.E + e) : zero16();
      pr[1][k] = pok ? load16(dptL + (p0 + l) * a.E + e) : zero16();
      const int first = 8 * (k * kThreads + tid);
      // a piece of r may straddle the end of the array, by whole values
      rv[k] = zero16();
      if (first < nr) {
        if ((int64_t)(first + 8) <= left * R2) rv[k] = load16(rr + p0 * R2 + first);
        else if ((int64_t)first < left * R2) {
          uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
          for (int j = 0; j < 8; ++j)   // (unrolled: w stays in registers)
            if ((int64_t)(first + j) < left * R2) w[j >> 1] |= (uint32_t)rr[p0 * R2 + first + j].v << (16 * (j & 1));
          rv[k] = make_uint4(w[0], w[1], w[2], w[3]);
        }
      }
    }
#pragma unroll
    for (int k = 0; k < kMaxZP; ++k) {
      const int o8 = wave + kWaves * k;
      zr[k] = o8 < ZP ? load16(a.dzt + (p0 + l) * a.Opad + 8 * o8) : zero16();
    }
  };
  // lane = position: the 8 values of a 16-byte piece go to 8 consecutive rows of a position-last block
  auto turn = [&](uint16_t* blk, uint4 v) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int j = 0; j < 8; ++j) blk[j * kPosStride + l] = (uint16_t)(w[j >> 1] >> (16 * (j & 1)));
  };

  if ((int)blockIdx.x < a.ntiles) fetch(blockIdx.x);
  for (int tile = blockIdx.x; tile < a.ntiles; tile += a.G) {
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const int row0 = 8 * (2 * wave + k);
      turn(xT + row0 * kPosStride, xr[k]);
      turn(pT + row0 * kPosStride, pr[0][k]);
      turn(pT + (kKC + row0) * kPosStride, pr[1][k]);
      const int first = 8 * (k * kThreads + tid);
      if (first < nr) {
        const uint32_t v[4] = {rv[k].x, rv[k].y, rv[k].z, rv[k].w};
        int p = rp[k], q = rq[k];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          if (p < kTP) rT[(q >= R ? rblk + (q - R) * kPosStride : q * kPosStride) + p] = (uint16_t)(v[j >> 1] >> (16 * (j & 1)));
          if (++q == R2) { q = 0; ++p; }
        }
      }
    }
#pragma unroll
    for (int k = 0; k < kMaxZP; ++k) {
      const int o8 = wave + kWaves * k;
      if (o8 < ZP) turn(zT + 8 * o8 * kPosStride, zr[k]);
    }
    __syncthreads();
    if (tile + a.G < a.ntiles) fetch(tile + a.G);
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      const int koff = 32 * ks + 8 * kb;
      const uint4 A0 = load16(zT + (16 * wave + mn) * kPosStride + koff);
      const uint4 A1 = wave + kWaves < MT ? load16(zT + (16 * (wave + kWaves) + mn) * kPosStride + koff) : zero16();
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) {
        const uint4 B = load16(xT + (16 * nt + mn) * kPosStride + koff);
        aw[0][nt] = mfma16(A0, B, aw[0][nt]);
        if (wave + kWaves < MT) aw[1][nt] = mfma16(A1, B, aw[1][nt]);
      }
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const uint4 Ap = load16(pT + (h * kKC + 16 * wave + mn) * kPosStride + koff);
#pragma unroll
        for (int nq = 0; nq < kMaxNQ1; ++nq)
          if (nq < NQ1) ar[h][nq] = mfma16(Ap, load16(rT + h * rblk + (16 * nq + mn) * kPosStride + koff), ar[h][nq]);
      }
    }
    __syncthreads();
  }

  // parts: D[4 kb + i][mn] of each accumulator
  float* out = a.part + ((int64_t)blockIdx.x * a.ne + ey) * (int64_t)(a.O + R2 + 2) * kKC;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int mt = wave + kWaves * h;
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int o = 16 * mt + 4 * kb + i;
        if (mt < MT && o < a.O) out[o * kKC + 16 * nt + mn] = aw[h][nt][i];
      }
#pragma unroll
    for (int nq = 0; nq < kMaxNQ1; ++nq) {
      const int q = 16 * nq + mn;
      const int row = q < R ? a.O + h * R + q : a.O + R2 + h;   // column R of the product is the bias gradient
      if (nq < NQ1 && q <= R) {
#pragma unroll
        for (int i = 0; i < 4; ++i) out[row * kKC + 16 * wave + 4 * kb + i] = ar[h][nq][i];
      }
    }
  }
}

// ------------------------------------------------------------------------------- backward, weights
// Grid (G, ne): workgroup (g, ey) adds up, over the tiles g, g+G, ..., the gradients of the weights
// that touch channels [64 ey, 64 ey + 64) and leaves them in part[g][ey][row][64]:
//   rows 0..O-1      dWx[o][.]      = sum_p dz[p][o] x[p][.]
//   rows O..O+R-1    dwT[.][q]      = sum_p dpreT[p][.] rT[p][q]      rows O+R..O+2R-1 the same for L
//   rows O+2R, +1    dbT[.], dbL[.] = sum_p dpre[p][.]
// LDS: xs[64][68], dpT[64][65], dpL[64][65], dzs[64][O4], rs[64][2R].  The loads of the next tile
// are under way while the sums of the current one are formed.
template <typename T, bool VEC>
__global__ __launch_bounds__(kThreads) void m2d_proj_bwd_weights_kernel(const ProjArgs a) {
  using TL = Tile<T, VEC>;
  extern __shared__ float smem[];
  const int O4 = a.O4;
  const int R = a.R, R2 = 2 * a.R;
  float* xs = smem;
  float* dpT = xs + kTP * kXS4;
  float* dpL = dpT + kTP * kXS;
  float* dzs = dpL + kTP * kXS;
  float* rs = dzs + kTP * O4;
  const int wave = wave_id(), lane = threadIdx.x & 63, tid = threadIdx.x;
  const int ey = blockIdx.y;
  const T* x = static_cast<const T*>(a.x);
  const T* rr = static_cast<const T*>(a.r);
  const T* dT = static_cast<const T*>(a.dT);
  const T* dL = static_cast<const T*>(a.dL);
  const T* ddT = static_cast<const T*>(a.ddT);
  const T* ddL = static_cast<const T*>(a.ddL);
  const bool given = a.dpre_given != 0;   // (uniform) ddT, ddL are dpre already
  const int64_t Pv = given ? 0 : a.P;     // rows of deltaT, deltaL to read: none then
  const int nmt = (O4 / 4) * 16;   // 4 x 4 blocks of dWx: (o4, e4), e4 fastest
  constexpr int kZQ = (kTP * ((2 * kMaxR + 3 * kN + 3) / 4) + kThreads - 1) / kThreads;   // float4 of dz per thread, at most
  constexpr int kRQ = (kTP * 2 * kMaxR + kThreads - 1) / kThreads;                        // elements of r per thread, at most
  const int nzq = kTP * O4 / 4, nrq = kTP * R2;

  float aw[2][16], ar[2][kMaxR / kWaves], ab[2] = {0.f, 0.f};
#pragma unroll
  for (int h = 0; h < 2; ++h) {
#pragma unroll
    for (int j = 0; j < 16; ++j) aw[h][j] = 0.f;
#pragma unroll
    for (int i = 0; i < kMaxR / kWaves; ++i) ar[h][i] = 0.f;
  }

  typename TL::Regs xr, gT, vT, gL, vL;
  float4 zq[kZQ];
  float rq[kRQ];
  auto fetch = [&](int tile) {
    const int64_t p0 = (int64_t)tile * kTP;
    TL::load(xr, x, p0, a.P, a.E, ey * kKC, tid);
    TL::load(gT, ddT, p0, a.P, a.E, ey * kKC, tid);
    TL::load(vT, dT, p0, Pv, a.E, ey * kKC, tid);
    TL::load(gL, ddL, p0, a.P, a.E, ey * kKC, tid);
    TL::load(vL, dL, p0, Pv, a.E, ey * kKC, tid);
    const int64_t left = a.P - p0;   // rows of the tile inside the array, if fewer than 64
    const float4* zsrc = reinterpret_cast<const float4*>(a.dz + p0 * O4);
#pragma unroll
    for (int k = 0; k < kZQ; ++k) {
      const int i = k * kThreads + tid;
      zq[k] = (i < nzq && (int64_t)(4 * i) < left * O4) ? zsrc[i] : make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int k = 0; k < kRQ; ++k) {
      const int i = k * kThreads + tid;
      rq[k] = (i < nrq && (int64_t)i < left * R2) ? ld(rr + p0 * R2 + i) : 0.f;
    }
  };

  if ((int)blockIdx.x < a.ntiles) fetch(blockIdx.x);
  for (int tile = blockIdx.x; tile < a.ntiles; tile += a.G) {
    TL::to_lds(xs, kXS4, tid, [&](int l, int j) { return TL::get(xr, l, j); });
    TL::to_lds(dpT, kXS, tid, [&](int l, int j) { return TL::get(gT, l, j) * (given ? 1.f : softplus_slope(TL::get(vT, l, j))); });
    TL::to_lds(dpL, kXS, tid, [&](int l, int j) { return TL::get(gL, l, j) * (given ? 1.f : softplus_slope(TL::get(vL, l, j))); });
#pragma unroll
    for (int k = 0; k < kZQ; ++k) {
      const int i = k * kThreads + tid;
      if (i < nzq) reinterpret_cast<float4*>(dzs)[i] = zq[k];
    }
#pragma unroll
    for (int k = 0; k < kRQ; ++k) {
      const int i = k * kThreads + tid;
      if (i < nrq) rs[i] = rq[k];
    }
    __syncthreads();
    if (tile + a.G < a.ntiles) fetch(tile + a.G);
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int mt = tid + kThreads * h;
      if (mt < nmt) {
        const float4* zp = reinterpret_cast<const float4*>(dzs + 4 * (mt >> 4));
        const float4* xp = reinterpret_cast<const float4*>(xs + 4 * (mt & 15));
#pragma unroll 4
        for (int c = 0; c < kTP; ++c) {
          const float4 z4 = zp[c * (O4 / 4)], x4 = xp[c * (kXS4 / 4)];
          const float zz[4] = {z4.x, z4.y, z4.z, z4.w}, xx[4] = {x4.x, x4.y, x4.z, x4.w};
#pragma unroll
          for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) aw[h][4 * i + j] = __builtin_fmaf(zz[i], xx[j], aw[h][4 * i + j]);
        }
      }
    }
    // dt weights: this thread's channel is `lane`, its ranks are wave, wave + 4, ...
#pragma unroll 2
    for (int c = 0; c < kTP; ++c) {
      const float tT = dpT[c * kXS + lane], tL = dpL[c * kXS + lane];
      const float* rc = rs + c * R2;
      if (wave == 0) { ab[0] += tT; ab[1] += tL; }
#pragma unroll
      for (int i = 0; i < kMaxR / kWaves; ++i) {
        const int q = wave + kWaves * i;
        if (q < R) {
          ar[0][i] = __builtin_fmaf(tT, rc[q], ar[0][i]);
          ar[1][i] = __builtin_fmaf(tL, rc[R + q], ar[1][i]);
        }
      }
    }
    __syncthreads();
  }

  float* out = a.part + ((int64_t)blockIdx.x * a.ne + ey) * (int64_t)(a.O + R2 + 2) * kKC;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int mt = tid + kThreads * h;
    if (mt < nmt) {
      const int o0 = 4 * (mt >> 4), e0 = 4 * (mt & 15);
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (o0 + i < a.O)
          *reinterpret_cast<float4*>(out + (o0 + i) * kKC + e0) = make_float4(aw[h][4 * i], aw[h][4 * i + 1], aw[h][4 * i + 2], aw[h][4 * i + 3]);
    }
  }
#pragma unroll
  for (int i = 0; i < kMaxR / kWaves; ++i) {
    const int q = wave + kWaves * i;
    if (q < R) {
      out[(a.O + q) * kKC + lane] = ar[0][i];
      out[(a.O + R + q) * kKC + lane] = ar[1][i];
    }
  }
  if (wave == 0) {
    out[(a.O + R2) * kKC + lane] = ab[0];
    out[(a.O + R2 + 1) * kKC + lane] = ab[1];
  }
}

// Sums the per-workgroup parts in a fixed order and scatters them to the five weight gradients.
// Grid (rows, ne), 1024 threads: 64 channels x 16 slices of the workgroup index.
constexpr int kRedSlices = 16;
__global__ __launch_bounds__(64 * kRedSlices) void m2d_proj_reduce_kernel(const ProjArgs a) {
  __shared__ float sums[kRedSlices][64];
  const int rows = a.O + 2 * a.R + 2;
  const int row = blockIdx.x, ey = blockIdx.y;
  const int el = threadIdx.x & 63, gs = threadIdx.x >> 6;
  const float* src = a.part + ((int64_t)ey * rows + row) * kKC + el;
  const int64_t gstride = (int64_t)a.ne * rows * kKC;
  float s = 0.f;
#pragma unroll 8
  for (int g = gs; g < a.G; g += kRedSlices) s += src[g * gstride];
  sums[gs][el] = s;
  __syncthreads();
  if (gs != 0) return;
#pragma unroll
  for (int k = 1; k < kRedSlices; ++k) s += sums[k][el];
  const int e = ey * kKC + el;
  if (e >= a.E) return;
  if (row < a.O) a.dWx[row * a.E + e] = s;
  else if (row < a.O + a.R) a.dwT[e * a.R + (row - a.O)] = s;
  else if (row < a.O + 2 * a.R) a.dwL[e * a.R + (row - a.O - a.R)] = s;
  else if (row == a.O + 2 * a.R) a.dbT[e] = s;
  else a.dbL[e] = s;
}

// ------------------------------------------------------------------------------- host
inline size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }
inline bool misaligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) != 0; }

struct ProjGeometry {
  int64_t P;
  int E, R, O, O4, Epad, Opad, Opad32, Rpad, ntiles, G, ne;
  bool vec;    // rows of the (P,E) arrays start on 16-byte boundaries
  bool mfma;   // bf16 and vec: products on the matrix cores
  // forward workspace
  size_t off_Wt, off_wTt, off_wLt, off_bTp, off_bLp, off_Wb, off_wTb, off_wLb, bytes_fwd;
  // backward workspace
  size_t off_Wp, off_wTp, off_wLp, off_wTtb, off_wLtb, off_WxTb, off_dz, off_dpt, off_part, bytes_bwd;
};

int check_proj(const m2d_desc* d, int R) {
  if (!d) return M2D_ERR_NULL_POINTER;
  if (d->B < 1 || d->H < 1 || d->W < 1 || d->E < 1 || d->N < 1 || R < 1) return M2D_ERR_BAD_SHAPE;
  if (d->N != kN || (d->dtype != M2D_F32 && d->dtype != M2D_BF16)) return M2D_ERR_UNSUPPORTED;   // (ckpt_interval is the scan's)
  if (d->flags & ~(M2D_FLAG_FLIP | M2D_FLAG_ROUND_WEIGHTS | M2D_FLAG_RAW_PARAMS | M2D_FLAG_PACKED_BC | M2D_FLAG_DPRE | M2D_FLAG_SPLIT_STATES | M2D_FLAG_WHOLE_STATES)) return M2D_ERR_UNSUPPORTED;
  if (R > kMaxR || d->E > 4096) return M2D_ERR_UNSUPPORTED;
  if ((int64_t)d->B * d->H * d->W >= ((int64_t)1 << 31) * kTP) return M2D_ERR_UNSUPPORTED;   // tiles counted in 32 bits
  return M2D_OK;
}

ProjGeometry proj_geometry(const m2d_desc* d, int R) {
  ProjGeometry g;
  g.P = (int64_t)d->B * d->H * d->W;
  g.E = d->E; g.R = R; g.O = 2 * R + 3 * kN;
  g.O4 = (g.O + 3) & ~3;
  g.Epad = (g.E + kKC - 1) / kKC * kKC;
  g.Opad = (g.O + 15) / 16 * 16;
  g.Opad32 = (g.O + 31) / 32 * 32;
  g.Rpad = (R + 15) / 16 * 16;
  g.ntiles = (int)((g.P + kTP - 1) / kTP);
  g.ne = g.Epad / kKC;
  g.vec = d->E % (d->dtype == M2D_F32 ? 4 : 8) == 0;
  g.mfma = g.vec && d->dtype == M2D_BF16;
  const int want = 512 / g.ne > 0 ? 512 / g.ne : 1;   // about two workgroups per compute unit in all
  g.G = g.ntiles < want ? g.ntiles : want;
  size_t o = 0;
  g.off_Wt = o; o += align256((size_t)g.Epad * g.Opad * 4);
  g.off_wTt = o; o += align256((size_t)R * g.Epad * 4);
  g.off_wLt = o; o += align256((size_t)R * g.Epad * 4);
  g.off_bTp = o; o += align256((size_t)g.Epad * 4);
  g.off_bLp = o; o += align256((size_t)g.Epad * 4);
  g.off_Wb = o; o += align256((size_t)g.Opad * g.Epad * 2);
  g.off_wTb = o; o += align256((size_t)g.Epad * 32 * 2);
  g.off_wLb = o; o += align256((size_t)g.Epad * 32 * 2);
  g.bytes_fwd = o;
  o = 0;
  g.off_Wp = o; o += align256((size_t)g.O * g.Epad * 4);
  g.off_wTp = o; o += align256((size_t)g.Epad * g.Rpad * 4);
  g.off_wLp = o; o += align256((size_t)g.Epad * g.Rpad * 4);
  g.off_wTtb = o; o += align256((size_t)g.Rpad * g.Epad * 2);
  g.off_wLtb = o; o += align256((size_t)g.Rpad * g.Epad * 2);
  g.off_WxTb = o; o += align256((size_t)g.Epad * g.Opad32 * 2);
  if (g.mfma) {   // dz and dpre as bf16 blocks per tile
    g.off_dz = o; o += align256((size_t)g.ntiles * kTP * g.Opad * 2);
    g.off_dpt = o; o += align256((size_t)2 * g.ntiles * kTP * g.E * 2);
  } else {
    g.off_dz = o; o += align256((size_t)g.P * g.O4 * 4);
    g.off_dpt = o;
  }
  g.off_part = o; o += align256((size_t)g.G * g.ne * (g.O + 2 * R + 2) * kKC * 4);
  g.bytes_bwd = o;
  return g;
}

void fill(ProjArgs& a, const ProjGeometry& g) {
  a.P = g.P; a.E = g.E; a.R = g.R; a.O = g.O; a.O4 = g.O4; a.Epad = g.Epad; a.Opad = g.Opad; a.Opad32 = g.Opad32; a.Rpad = g.Rpad;
  a.ntiles = g.ntiles; a.G = g.G; a.ne = g.ne;
}

inline bool launched() { return hipGetLastError() == hipSuccess; }

constexpr int kMaxLdsWeights = (kTP * kXS4 + 2 * kTP * kXS + kTP * ((2 * kMaxR + 3 * kN + 3) & ~3) + kTP * 2 * kMaxR) * 4;

template <typename T, bool VEC>
bool allow_lds_weights() {
  // more than 64 KB of dynamic LDS has to be allowed once per device (one bit per device ordinal)
  static std::atomic<uint64_t> seen{0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return false;
  const uint64_t bit = 1ull << (dev & 63);
  if (seen.load(std::memory_order_relaxed) & bit) return true;
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(&m2d_proj_bwd_weights_kernel<T, VEC>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLdsWeights) != hipSuccess)
    return false;
  seen.fetch_or(bit, std::memory_order_relaxed);
  return true;
}

int run_proj_fwd_mfma(const ProjGeometry& g, const ProjArgs& a, hipStream_t st) {
  const size_t lds = (size_t)kWaves * (16 * kStageStride * 4 + 2 * 16 * kLowStride * 2);
  hipLaunchKernelGGL(m2d_proj_fwd_mfma_kernel, dim3(g.ntiles), dim3(kThreads), lds, st, a);
  return launched() ? M2D_OK : M2D_ERR_HIP;
}

template <typename T, bool VEC>
int run_proj_fwd(const ProjGeometry& g, const ProjArgs& a, hipStream_t st) {
  const size_t lds = (size_t)(2 * kTP * kXS + kTP * (g.O + 1)) * 4;
  hipLaunchKernelGGL((m2d_proj_fwd_kernel<T, VEC>), dim3(g.ntiles), dim3(kThreads), lds, st, a);
  return launched() ? M2D_OK : M2D_ERR_HIP;
}

template <typename T, bool VEC>
int run_proj_bwd(const ProjGeometry& g, const ProjArgs& a, hipStream_t st) {
  if (g.mfma) {
    const size_t lds_data = (size_t)kWaves * (16 * kStageStride * 4 + 16 * (g.Opad32 + 8) * 2);
    hipLaunchKernelGGL(m2d_proj_bwd_data_mfma_kernel, dim3(g.ntiles), dim3(kThreads), lds_data, st, a);
    if (!launched()) return M2D_ERR_HIP;
    const size_t lds_w = (size_t)(3 * kKC + g.Opad + 2 * 16 * ((g.R + 1 + 15) / 16)) * kPosStride * 2;
    hipLaunchKernelGGL(m2d_proj_bwd_weights_mfma_kernel, dim3(g.G, g.ne), dim3(kThreads), lds_w, st, a);
    if (!launched()) return M2D_ERR_HIP;
    hipLaunchKernelGGL(m2d_proj_reduce_kernel, dim3(g.O + 2 * g.R + 2, g.ne), dim3(64 * kRedSlices), 0, st, a);
    return launched() ? M2D_OK : M2D_ERR_HIP;
  } else {
    const size_t lds_data = (size_t)(2 * kTP * kXS + kTP * (g.O + 1)) * 4;
    hipLaunchKernelGGL((m2d_proj_bwd_data_kernel<T, VEC>), dim3(g.ntiles), dim3(kThreads), lds_data, st, a);
  }
  if (!launched()) return M2D_ERR_HIP;
  const size_t lds_w = (size_t)(kTP * kXS4 + 2 * kTP * kXS + kTP * g.O4 + kTP * 2 * g.R) * 4;
  if (!allow_lds_weights<T, VEC>()) return M2D_ERR_HIP;
  hipLaunchKernelGGL((m2d_proj_bwd_weights_kernel<T, VEC>), dim3(g.G, g.ne), dim3(kThreads), lds_w, st, a);
  if (!launched()) return M2D_ERR_HIP;
  hipLaunchKernelGGL(m2d_proj_reduce_kernel, dim3(g.O + 2 * g.R + 2, g.ne), dim3(64 * kRedSlices), 0, st, a);
  return launched() ? M2D_OK : M2D_ERR_HIP;
}

}  // namespace

extern "C" {

size_t m2d_proj_workspace_bytes(const m2d_desc* desc, int dt_rank, int pass) {
  if (check_proj(desc, dt_rank) != M2D_OK || (pass != M2D_PASS_FWD && pass != M2D_PASS_BWD)) return 0;
  const ProjGeometry g = proj_geometry(desc, dt_rank);
  return pass == M2D_PASS_FWD ? g.bytes_fwd : g.bytes_bwd;
}

int m2d_proj_fwd(const m2d_desc* desc, int dt_rank, const void* x, const float* x_proj_w, const float* dt_projT_w,
                 const float* dt_projT_b, const float* dt_projL_w, const float* dt_projL_b, void* lowrank,
                 void* deltaT, void* deltaL, void* BT, void* BL, void* C, void* workspace, size_t workspace_bytes,
                 void* stream) {
  int rc = check_proj(desc, dt_rank);
  if (rc) return rc;
  const bool packed = (desc->flags & M2D_FLAG_PACKED_BC) != 0;   // B_T takes the records, B_L and C are not written
  const void* req[] = {x, x_proj_w, dt_projT_w, dt_projT_b, dt_projL_w, dt_projL_b, lowrank, deltaT, deltaL, BT,
                       packed ? BT : BL, packed ? BT : C, workspace};
  for (const void* q : req) if (!q) return M2D_ERR_NULL_POINTER;
  for (const void* q : req) if (misaligned(q, 16)) return M2D_ERR_MISALIGNED;
  if (misaligned(workspace, 256)) return M2D_ERR_MISALIGNED;
  const ProjGeometry g = proj_geometry(desc, dt_rank);
  if (workspace_bytes < g.bytes_fwd) return M2D_ERR_WORKSPACE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  char* ws = static_cast<char*>(workspace);
  PackArgs k = {};
  k.Wx = x_proj_w; k.wT = dt_projT_w; k.bT = dt_projT_b; k.wL = dt_projL_w; k.bL = dt_projL_b;
  k.Wt = reinterpret_cast<float*>(ws + g.off_Wt);
  k.wTt = reinterpret_cast<float*>(ws + g.off_wTt);
  k.wLt = reinterpret_cast<float*>(ws + g.off_wLt);
  k.bTp = reinterpret_cast<float*>(ws + g.off_bTp);
  k.bLp = reinterpret_cast<float*>(ws + g.off_bLp);
  if (g.mfma) {   // the matrix-core kernel reads the bf16 set
    k.Wt = nullptr;
    k.Wb = reinterpret_cast<uint16_t*>(ws + g.off_Wb);
    k.wTb = reinterpret_cast<uint16_t*>(ws + g.off_wTb);
    k.wLb = reinterpret_cast<uint16_t*>(ws + g.off_wLb);
  }
  k.E = g.E; k.R = g.R; k.O = g.O; k.Epad = g.Epad; k.Opad = g.Opad; k.Opad32 = g.Opad32; k.Rpad = g.Rpad;
  k.round = (desc->flags & M2D_FLAG_ROUND_WEIGHTS) && desc->dtype == M2D_BF16;
  const int n = g.Epad * (g.Opad > 32 ? g.Opad : 32);   // the largest forward copy
  hipLaunchKernelGGL(m2d_proj_pack_kernel, dim3((n + 255) / 256), dim3(256), 0, st, k);
  if (!launched()) return M2D_ERR_HIP;
  ProjArgs a = {};
  fill(a, g);
  a.x = x; a.Wt = k.Wt; a.wTt = k.wTt; a.wLt = k.wLt; a.bTp = k.bTp; a.bLp = k.bLp;
  a.Wb = k.Wb; a.wTb = k.wTb; a.wLb = k.wLb;
  a.r_out = lowrank; a.dT_out = deltaT; a.dL_out = deltaL; a.BT_out = BT; a.BL_out = BL; a.C_out = C;
  a.bc_packed = packed ? static_cast<float*>(BT) : nullptr;
  if (desc->dtype == M2D_F32) return g.vec ? run_proj_fwd<float, true>(g, a, st) : run_proj_fwd<float, false>(g, a, st);
  return g.mfma ? run_proj_fwd_mfma(g, a, st) : run_proj_fwd<bf16_t, false>(g, a, st);
}

int m2d_proj_bwd(const m2d_desc* desc, int dt_rank, const void* x, const void* lowrank, const void* deltaT,
                 const void* deltaL, const float* x_proj_w, const float* dt_projT_w, const float* dt_projL_w,
                 const void* d_deltaT, const void* d_deltaL, const void* d_BT, const void* d_BL, const void* d_C,
                 void* dx, float* d_x_proj_w, float* d_dt_projT_w, float* d_dt_projT_b, float* d_dt_projL_w,
                 float* d_dt_projL_b, void* workspace, size_t workspace_bytes, void* stream) {
  return m2d_proj_bwd_parts(desc, dt_rank, 0, x, lowrank, deltaT, deltaL, x_proj_w, dt_projT_w, dt_projL_w, d_deltaT, d_deltaL, d_BT, d_BL,
                            d_C, dx, d_x_proj_w, d_dt_projT_w, d_dt_projT_b, d_dt_projL_w, d_dt_projL_b, workspace, workspace_bytes, stream);
}

int m2d_proj_bwd_parts(const m2d_desc* desc, int dt_rank, int sum_parts, const void* x, const void* lowrank, const void* deltaT,
                       const void* deltaL, const float* x_proj_w, const float* dt_projT_w, const float* dt_projL_w,
                       const void* d_deltaT, const void* d_deltaL, const void* d_BT, const void* d_BL, const void* d_C,
                       void* dx, float* d_x_proj_w, float* d_dt_projT_w, float* d_dt_projT_b, float* d_dt_projL_w,
                       float* d_dt_projL_b, void* workspace, size_t workspace_bytes, void* stream) {
  int rc = check_proj(desc, dt_rank);
  if (rc) return rc;
  if (sum_parts < 0) return M2D_ERR_BAD_SHAPE;
  if (sum_parts > 0 && !proj_geometry(desc, dt_rank).mfma) return M2D_ERR_UNSUPPORTED;
  const bool given = (desc->flags & M2D_FLAG_DPRE) != 0;   // d_deltaT, d_deltaL are dpre: deltaT, deltaL are not read
  const void* req[] = {x, lowrank, x_proj_w, dt_projT_w, dt_projL_w, d_deltaT, d_deltaL, d_BT, sum_parts ? d_BT : d_BL, sum_parts ? d_BT : d_C,
                       dx, d_x_proj_w, d_dt_projT_w, d_dt_projT_b, d_dt_projL_w, d_dt_projL_b, workspace};
  for (const void* q : req) if (!q) return M2D_ERR_NULL_POINTER;
  if (!given && (!deltaT || !deltaL)) return M2D_ERR_NULL_POINTER;
  for (const void* q : req) if (misaligned(q, 16)) return M2D_ERR_MISALIGNED;
  if (!given && (misaligned(deltaT, 16) || misaligned(deltaL, 16))) return M2D_ERR_MISALIGNED;
  if (misaligned(workspace, 256)) return M2D_ERR_MISALIGNED;
  const ProjGeometry g = proj_geometry(desc, dt_rank);
  if (workspace_bytes < g.bytes_bwd) return M2D_ERR_WORKSPACE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  char* ws = static_cast<char*>(workspace);
  PackArgs k = {};
  k.Wx = x_proj_w; k.wT = dt_projT_w; k.wL = dt_projL_w;
  k.Wp = reinterpret_cast<float*>(ws + g.off_Wp);
  k.wTp = reinterpret_cast<float*>(ws + g.off_wTp);
  k.wLp = reinterpret_cast<float*>(ws + g.off_wLp);
  if (g.mfma) {   // the data kernel reads the bf16 set; the weight-gradient kernel needs no weights
    k.Wp = nullptr;
    k.wTtb = reinterpret_cast<uint16_t*>(ws + g.off_wTtb);
    k.wLtb = reinterpret_cast<uint16_t*>(ws + g.off_wLtb);
    k.WxTb = reinterpret_cast<uint16_t*>(ws + g.off_WxTb);
  }
  k.E = g.E; k.R = g.R; k.O = g.O; k.Epad = g.Epad; k.Opad = g.Opad; k.Opad32 = g.Opad32; k.Rpad = g.Rpad;
  k.round = (desc->flags & M2D_FLAG_ROUND_WEIGHTS) && desc->dtype == M2D_BF16;
  int n = g.Opad32 * g.Epad;
  if (g.Epad * g.Rpad > n) n = g.Epad * g.Rpad;
  hipLaunchKernelGGL(m2d_proj_pack_kernel, dim3((n + 255) / 256), dim3(256), 0, st, k);
  if (!launched()) return M2D_ERR_HIP;
  ProjArgs a = {};
  fill(a, g);
  a.x = x; a.r = lowrank; a.dT = deltaT; a.dL = deltaL; a.dpre_given = given ? 1 : 0; a.sum_parts = sum_parts;
  a.ddT = d_deltaT; a.ddL = d_deltaL; a.dBT = d_BT; a.dBL = d_BL; a.dC = d_C; a.dx = dx;
  a.Wp = k.Wp; a.wTp = k.wTp; a.wLp = k.wLp;
  a.wTtb = k.wTtb; a.wLtb = k.wLtb; a.WxTb = k.WxTb;
  a.dz = reinterpret_cast<float*>(ws + g.off_dz);
  a.dzt = reinterpret_cast<uint16_t*>(ws + g.off_dz);
  a.dpt = reinterpret_cast<uint16_t*>(ws + g.off_dpt);
  a.part = reinterpret_cast<float*>(ws + g.off_part);
  a.dWx = d_x_proj_w; a.dwT = d_dt_projT_w; a.dbT = d_dt_projT_b; a.dwL = d_dt_projL_w; a.dbL = d_dt_projL_b;
  if (desc->dtype == M2D_F32) return g.vec ? run_proj_bwd<float, true>(g, a, st) : run_proj_bwd<float, false>(g, a, st);
  return g.vec ? run_proj_bwd<bf16_t, true>(g, a, st) : run_proj_bwd<bf16_t, false>(g, a, st);
}

}  // extern "C"

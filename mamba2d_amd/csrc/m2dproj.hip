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
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);  // NaN
  u += 0x7fffu + ((u >> 16) & 1u);                                            // round to nearest even
  return (uint16_t)(u >> 16);
}
__device__ __forceinline__ void st(float* p, float v) { *p = v; }
__device__ __forceinline__ void st(bf16_t* p, float v) { p->v = f32_to_bf16_bits(v); }
// the value a tensor of type T would hold
__device__ __forceinline__ float as_stored(float v, const float*) { return v; }
__device__ __forceinline__ float as_stored(float v, const bf16_t*) { return __uint_as_float((uint32_t)f32_to_bf16_bits(v) << 16); }

// softplus with torch's defaults (beta 1, threshold 20)
__device__ __forceinline__ float softplus(float v) { return v > 20.f ? v : log1pf(expf(v)); }
// d softplus / d pre, from the softplus value: sigmoid(pre) = 1 - exp(-softplus(pre))
__device__ __forceinline__ float softplus_slope(float delta) { return -expm1f(-delta); }

struct ProjArgs {
  // activations, (P, .) row-major, element type T
  const void *x, *r, *dT, *dL;           // x (P,E); r (P,2R) = low-rank inputs of the two dt projections; delta (P,E)
  const void *ddT, *ddL, *dBT, *dBL, *dC;
  void *r_out, *dT_out, *dL_out, *BT_out, *BL_out, *C_out, *dx;
  // weights, fp32
  const float *bT, *bL;                  // (E)
  const float *wT, *wL;                  // (E,R) as given
  const float *Wt;                       // [Epad][Opad]   Wx transposed, zero padded
  const float *Wp;                       // [O][Epad]      Wx, rows padded
  const float *wTp, *wLp;                // [Epad][Rpad]   dt weights, rows padded
  float* dz;                             // (P,O) fp32
  float* part;                           // per-workgroup sums of the weight gradients
  float *dWx, *dwT, *dbT, *dwL, *dbL;    // outputs of the reduction
  int64_t P;
  int E, R, O, Epad, Opad, Rpad;
  int ntiles, G, ne;
};

// Packed weights are read through the constant address space: they were written by an earlier
// launch, and a wave-uniform load from that space is a scalar load whatever the kernel stores.
typedef const __attribute__((address_space(4))) float* const_floats;
__device__ __forceinline__ const_floats as_const(const float* p) { return (const_floats)(uintptr_t)p; }

__device__ __forceinline__ int wave_id() { return __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)); }

// ------------------------------------------------------------------------------- weights
// Padded copies of the weights (zero where padded).  One thread per element of the largest copy.
__global__ void m2d_proj_pack_kernel(const float* __restrict__ Wx, const float* __restrict__ wT, const float* __restrict__ wL,
                                     float* __restrict__ Wt, float* __restrict__ Wp, float* __restrict__ wTp, float* __restrict__ wLp,
                                     int E, int R, int O, int Epad, int Opad, int Rpad) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (Wt && i < Epad * Opad) {
    const int e = i / Opad, o = i - e * Opad;
    Wt[i] = (e < E && o < O) ? Wx[o * E + e] : 0.f;
  }
  if (Wp && i < O * Epad) {
    const int o = i / Epad, e = i - o * Epad;
    Wp[i] = e < E ? Wx[o * E + e] : 0.f;
  }
  if (wTp && i < Epad * Rpad) {
    const int e = i / Rpad, q = i - e * Rpad;
    const bool ok = e < E && q < R;
    wTp[i] = ok ? wT[e * R + q] : 0.f;
    wLp[i] = ok ? wL[e * R + q] : 0.f;
  }
}

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
// One workgroup per tile of 64 positions.  LDS: xs[64][65] (a chunk of x), zs[64][O+1] (z).
template <typename T>
__global__ __launch_bounds__(kThreads) void m2d_proj_fwd_kernel(const ProjArgs a) {
  extern __shared__ float smem[];
  float* xs = smem;
  float* zs = smem + kTP * kXS;
  const int zst = a.O + 1;
  const int wave = wave_id(), lane = threadIdx.x & 63;
  const int64_t p0 = (int64_t)blockIdx.x * kTP;
  const T* x = static_cast<const T*>(a.x);
  const int nOC = a.Opad / 16;

  float acc[kMaxRounds][16];
#pragma unroll
  for (int rd = 0; rd < kMaxRounds; ++rd)
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[rd][j] = 0.f;

  for (int kc = 0; kc < a.Epad / kKC; ++kc) {
    const int e = kc * kKC + lane;
    for (int c = wave; c < kTP; c += kWaves) {
      const int64_t p = p0 + c;
      xs[c * kXS + lane] = (p < a.P && e < a.E) ? ld(x + p * a.E + e) : 0.f;
    }
    __syncthreads();
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

  // ---- outputs, a row of the tile per wave at a time (rows are contiguous in memory)
  const int R = a.R, R2 = 2 * a.R;
  T* r_out = static_cast<T*>(a.r_out);
  T* dT_out = static_cast<T*>(a.dT_out);
  T* dL_out = static_cast<T*>(a.dL_out);
  for (int c = wave; c < kTP; c += kWaves) {
    const int64_t p = p0 + c;
    if (p >= a.P) break;   // uniform
    const float* z = zs + c * zst;
    for (int q = lane; q < R2; q += 64) st(r_out + p * R2 + q, z[q]);
    if (lane < 3 * kN) {
      T* out = static_cast<T*>(lane < kN ? a.BT_out : (lane < 2 * kN ? a.BL_out : a.C_out));
      st(out + p * kN + (lane & (kN - 1)), z[R2 + lane]);
    }
    for (int e = lane; e < a.E; e += 64) {
      float preT = a.bT[e], preL = a.bL[e];
      const float* wt = a.wT + e * R;
      const float* wl = a.wL + e * R;
      for (int q = 0; q < R; ++q) {
        // the dt projections see the low-rank inputs as the tensor holds them
        preT = __builtin_fmaf(as_stored(z[q], r_out), wt[q], preT);
        preL = __builtin_fmaf(as_stored(z[R + q], r_out), wl[q], preL);
      }
      st(dT_out + p * a.E + e, softplus(preT));
      st(dL_out + p * a.E + e, softplus(preL));
    }
  }
}

// ------------------------------------------------------------------------------- backward, data
// One workgroup per tile.  LDS: dps[2][64][65] (chunks of dpreT, dpreL; reused for the dx tile),
// dzs[64][O+1].  Writes dz (P,O) for the weight-gradient kernel and adds dz Wx to dx.
template <typename T>
__global__ __launch_bounds__(kThreads) void m2d_proj_bwd_data_kernel(const ProjArgs a) {
  extern __shared__ float smem[];
  float* dps = smem;
  float* dzs = smem + 2 * kTP * kXS;
  const int zst = a.O + 1;
  const int wave = wave_id(), lane = threadIdx.x & 63;
  const int64_t p0 = (int64_t)blockIdx.x * kTP;
  const int R = a.R, R2 = 2 * a.R;
  const int nRC = a.Rpad / 16;   // 16-wide chunks of one dt weight; 2*nRC chunks in all (T then L)
  const T* dT = static_cast<const T*>(a.dT);
  const T* dL = static_cast<const T*>(a.dL);
  const T* ddT = static_cast<const T*>(a.ddT);
  const T* ddL = static_cast<const T*>(a.ddL);

  float acc[kMaxRounds][16];
#pragma unroll
  for (int rd = 0; rd < kMaxRounds; ++rd)
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[rd][j] = 0.f;

  for (int kc = 0; kc < a.Epad / kKC; ++kc) {
    const int e = kc * kKC + lane;
    for (int c = wave; c < kTP; c += kWaves) {
      const int64_t p = p0 + c;
      float vT = 0.f, vL = 0.f;
      if (p < a.P && e < a.E) {
        const int64_t i = p * a.E + e;
        vT = ld(ddT + i) * softplus_slope(ld(dT + i));
        vL = ld(ddL + i) * softplus_slope(ld(dL + i));
      }
      dps[c * kXS + lane] = vT;
      dps[kTP * kXS + c * kXS + lane] = vL;
    }
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
  for (int c = wave; c < kTP; c += kWaves) {
    const int64_t p = p0 + c;
    if (lane < 3 * kN) {
      const T* src = static_cast<const T*>(lane < kN ? a.dBT : (lane < 2 * kN ? a.dBL : a.dC));
      dzs[c * zst + R2 + lane] = p < a.P ? ld(src + p * kN + (lane & (kN - 1))) : 0.f;
    }
  }
  __syncthreads();

  for (int c = wave; c < kTP; c += kWaves) {
    const int64_t p = p0 + c;
    if (p >= a.P) break;   // uniform
    for (int o = lane; o < a.O; o += 64) a.dz[p * a.O + o] = dzs[c * zst + o];
  }

  // ---- dx += dz Wx, 64 channels at a time (16 per wave), through LDS for row-wise stores
  T* dx = static_cast<T*>(a.dx);
  float* outs = dps;
  for (int eg = 0; eg < a.Epad / kKC; ++eg) {
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
#pragma unroll
    for (int j = 0; j < 16; ++j) outs[lane * kXS + wave * 16 + j] = s[j];
    __syncthreads();
    const int e = eg * kKC + lane;
    for (int c = wave; c < kTP; c += kWaves) {
      const int64_t p = p0 + c;
      if (p < a.P && e < a.E) st(dx + p * a.E + e, ld(dx + p * a.E + e) + outs[c * kXS + lane]);
    }
    __syncthreads();
  }
}

// ------------------------------------------------------------------------------- backward, weights
// Grid (G, ne): workgroup (g, ey) adds up, over the tiles g, g+G, ..., the gradients of the weights
// that touch channels [64 ey, 64 ey + 64) and leaves them in part[g][ey][row][64]:
//   rows 0..O-1      dWx[o][.]      = sum_p dz[p][o] x[p][.]
//   rows O..O+R-1    dwT[.][q]      = sum_p dpreT[p][.] rT[p][q]      rows O+R..O+2R-1 the same for L
//   rows O+2R, +1    dbT[.], dbL[.] = sum_p dpre[p][.]
// LDS: xs[64][68], dpT[64][65], dpL[64][65], dzs[64][O4], rs[64][2R+1].
template <typename T>
__global__ __launch_bounds__(kThreads) void m2d_proj_bwd_weights_kernel(const ProjArgs a) {
  extern __shared__ float smem[];
  const int O4 = (a.O + 3) & ~3;
  const int R = a.R, R2 = 2 * a.R, rst = R2 + 1;
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
  const int nmt = (O4 / 4) * 16;   // 4 x 4 blocks of dWx: (o4, e4), e4 fastest

  float aw[2][16], ar[2][kMaxR / kWaves], ab[2] = {0.f, 0.f};
#pragma unroll
  for (int h = 0; h < 2; ++h) {
#pragma unroll
    for (int j = 0; j < 16; ++j) aw[h][j] = 0.f;
#pragma unroll
    for (int i = 0; i < kMaxR / kWaves; ++i) ar[h][i] = 0.f;
  }

  for (int tile = blockIdx.x; tile < a.ntiles; tile += a.G) {
    const int64_t p0 = (int64_t)tile * kTP;
    const int e = ey * kKC + lane;
    for (int c = wave; c < kTP; c += kWaves) {
      const int64_t p = p0 + c;
      const bool row = p < a.P;
      float xv = 0.f, vT = 0.f, vL = 0.f;
      if (row && e < a.E) {
        const int64_t i = p * a.E + e;
        xv = ld(x + i);
        vT = ld(ddT + i) * softplus_slope(ld(dT + i));
        vL = ld(ddL + i) * softplus_slope(ld(dL + i));
      }
      xs[c * kXS4 + lane] = xv;
      dpT[c * kXS + lane] = vT;
      dpL[c * kXS + lane] = vL;
      for (int o = lane; o < O4; o += 64) dzs[c * O4 + o] = (row && o < a.O) ? a.dz[p * a.O + o] : 0.f;
      for (int q = lane; q < R2; q += 64) rs[c * rst + q] = row ? ld(rr + p * R2 + q) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int mt = tid + kThreads * h;
      if (mt < nmt) {
        const float4* zq = reinterpret_cast<const float4*>(dzs + 4 * (mt >> 4));
        const float4* xq = reinterpret_cast<const float4*>(xs + 4 * (mt & 15));
#pragma unroll 4
        for (int c = 0; c < kTP; ++c) {
          const float4 z4 = zq[c * (O4 / 4)], x4 = xq[c * (kXS4 / 4)];
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
      const float vT = dpT[c * kXS + lane], vL = dpL[c * kXS + lane];
      const float* rq = rs + c * rst;
      if (wave == 0) { ab[0] += vT; ab[1] += vL; }
#pragma unroll
      for (int i = 0; i < kMaxR / kWaves; ++i) {
        const int q = wave + kWaves * i;
        if (q < R) {
          ar[0][i] = __builtin_fmaf(vT, rq[q], ar[0][i]);
          ar[1][i] = __builtin_fmaf(vL, rq[R + q], ar[1][i]);
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

// Sums the per-workgroup parts in workgroup order and scatters them to the five weight gradients.
__global__ void m2d_proj_reduce_kernel(const ProjArgs a) {
  const int rows = a.O + 2 * a.R + 2;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= rows * a.E) return;
  const int row = i / a.E, e = i - row * a.E;
  const int ey = e / kKC, el = e - ey * kKC;
  const float* src = a.part + ((int64_t)ey * rows + row) * kKC + el;
  const int64_t gstride = (int64_t)a.ne * rows * kKC;
  float s = 0.f;
  for (int g = 0; g < a.G; ++g) s += src[g * gstride];
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
  int E, R, O, Epad, Opad, Rpad, ntiles, G, ne;
  size_t off_Wt, off_Wp, off_wTp, off_wLp, off_dz, off_part, bytes_fwd, bytes_bwd;
};

int check_proj(const m2d_desc* d, int R) {
  if (!d) return M2D_ERR_NULL_POINTER;
  if (d->B < 1 || d->H < 1 || d->W < 1 || d->E < 1 || d->N < 1 || R < 1) return M2D_ERR_BAD_SHAPE;
  if (d->N != kN || (d->dtype != M2D_F32 && d->dtype != M2D_BF16) || d->reserved != 0) return M2D_ERR_UNSUPPORTED;
  if (R > kMaxR || d->E > 4096) return M2D_ERR_UNSUPPORTED;
  if ((int64_t)d->B * d->H * d->W >= ((int64_t)1 << 31) * kTP) return M2D_ERR_UNSUPPORTED;   // tiles counted in 32 bits
  return M2D_OK;
}

ProjGeometry proj_geometry(const m2d_desc* d, int R) {
  ProjGeometry g;
  g.P = (int64_t)d->B * d->H * d->W;
  g.E = d->E; g.R = R; g.O = 2 * R + 3 * kN;
  g.Epad = (g.E + kKC - 1) / kKC * kKC;
  g.Opad = (g.O + 15) / 16 * 16;
  g.Rpad = (R + 15) / 16 * 16;
  g.ntiles = (int)((g.P + kTP - 1) / kTP);
  g.ne = g.Epad / kKC;
  const int want = 512 / g.ne > 0 ? 512 / g.ne : 1;   // about two workgroups per compute unit in all
  g.G = g.ntiles < want ? g.ntiles : want;
  size_t o = 0;
  g.off_Wt = o; o += align256((size_t)g.Epad * g.Opad * 4);
  g.bytes_fwd = o;
  o = 0;
  g.off_Wp = o; o += align256((size_t)g.O * g.Epad * 4);
  g.off_wTp = o; o += align256((size_t)g.Epad * g.Rpad * 4);
  g.off_wLp = o; o += align256((size_t)g.Epad * g.Rpad * 4);
  g.off_dz = o; o += align256((size_t)g.P * g.O * 4);
  g.off_part = o; o += align256((size_t)g.G * g.ne * (g.O + 2 * R + 2) * kKC * 4);
  g.bytes_bwd = o;
  return g;
}

void fill(ProjArgs& a, const ProjGeometry& g) {
  a.P = g.P; a.E = g.E; a.R = g.R; a.O = g.O; a.Epad = g.Epad; a.Opad = g.Opad; a.Rpad = g.Rpad;
  a.ntiles = g.ntiles; a.G = g.G; a.ne = g.ne;
}

inline bool launched() { return hipGetLastError() == hipSuccess; }

constexpr int kMaxLdsWeights = (kTP * kXS4 + 2 * kTP * kXS + kTP * ((2 * kMaxR + 3 * kN + 3) & ~3) + kTP * (2 * kMaxR + 1)) * 4;

template <typename T>
bool allow_lds_weights() {
  static bool done = false;   // idempotent, the value never changes
  if (!done) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&m2d_proj_bwd_weights_kernel<T>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLdsWeights) != hipSuccess)
      return false;
    done = true;
  }
  return true;
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
  const void* req[] = {x, x_proj_w, dt_projT_w, dt_projT_b, dt_projL_w, dt_projL_b, lowrank, deltaT, deltaL, BT, BL, C, workspace};
  for (const void* q : req) if (!q) return M2D_ERR_NULL_POINTER;
  for (const void* q : req) if (misaligned(q, 16)) return M2D_ERR_MISALIGNED;
  if (misaligned(workspace, 256)) return M2D_ERR_MISALIGNED;
  const ProjGeometry g = proj_geometry(desc, dt_rank);
  if (workspace_bytes < g.bytes_fwd) return M2D_ERR_WORKSPACE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  char* ws = static_cast<char*>(workspace);
  float* Wt = reinterpret_cast<float*>(ws + g.off_Wt);
  const int n = g.Epad * g.Opad;
  hipLaunchKernelGGL(m2d_proj_pack_kernel, dim3((n + 255) / 256), dim3(256), 0, st, x_proj_w, dt_projT_w, dt_projL_w, Wt,
                     (float*)nullptr, (float*)nullptr, (float*)nullptr, g.E, g.R, g.O, g.Epad, g.Opad, g.Rpad);
  if (!launched()) return M2D_ERR_HIP;
  ProjArgs a = {};
  fill(a, g);
  a.x = x; a.Wt = Wt; a.wT = dt_projT_w; a.wL = dt_projL_w; a.bT = dt_projT_b; a.bL = dt_projL_b;
  a.r_out = lowrank; a.dT_out = deltaT; a.dL_out = deltaL; a.BT_out = BT; a.BL_out = BL; a.C_out = C;
  const size_t lds = (size_t)(kTP * kXS + kTP * (g.O + 1)) * 4;
  if (desc->dtype == M2D_F32)
    hipLaunchKernelGGL(m2d_proj_fwd_kernel<float>, dim3(g.ntiles), dim3(kThreads), lds, st, a);
  else
    hipLaunchKernelGGL(m2d_proj_fwd_kernel<bf16_t>, dim3(g.ntiles), dim3(kThreads), lds, st, a);
  return launched() ? M2D_OK : M2D_ERR_HIP;
}

int m2d_proj_bwd(const m2d_desc* desc, int dt_rank, const void* x, const void* lowrank, const void* deltaT,
                 const void* deltaL, const float* x_proj_w, const float* dt_projT_w, const float* dt_projL_w,
                 const void* d_deltaT, const void* d_deltaL, const void* d_BT, const void* d_BL, const void* d_C,
                 void* dx, float* d_x_proj_w, float* d_dt_projT_w, float* d_dt_projT_b, float* d_dt_projL_w,
                 float* d_dt_projL_b, void* workspace, size_t workspace_bytes, void* stream) {
  int rc = check_proj(desc, dt_rank);
  if (rc) return rc;
  const void* req[] = {x, lowrank, deltaT, deltaL, x_proj_w, dt_projT_w, dt_projL_w, d_deltaT, d_deltaL, d_BT, d_BL, d_C,
                       dx, d_x_proj_w, d_dt_projT_w, d_dt_projT_b, d_dt_projL_w, d_dt_projL_b, workspace};
  for (const void* q : req) if (!q) return M2D_ERR_NULL_POINTER;
  for (const void* q : req) if (misaligned(q, 16)) return M2D_ERR_MISALIGNED;
  if (misaligned(workspace, 256)) return M2D_ERR_MISALIGNED;
  const ProjGeometry g = proj_geometry(desc, dt_rank);
  if (workspace_bytes < g.bytes_bwd) return M2D_ERR_WORKSPACE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  char* ws = static_cast<char*>(workspace);
  float* Wp = reinterpret_cast<float*>(ws + g.off_Wp);
  float* wTp = reinterpret_cast<float*>(ws + g.off_wTp);
  float* wLp = reinterpret_cast<float*>(ws + g.off_wLp);
  int n = g.O * g.Epad;
  if (g.Epad * g.Rpad > n) n = g.Epad * g.Rpad;
  hipLaunchKernelGGL(m2d_proj_pack_kernel, dim3((n + 255) / 256), dim3(256), 0, st, x_proj_w, dt_projT_w, dt_projL_w,
                     (float*)nullptr, Wp, wTp, wLp, g.E, g.R, g.O, g.Epad, g.Opad, g.Rpad);
  if (!launched()) return M2D_ERR_HIP;
  ProjArgs a = {};
  fill(a, g);
  a.x = x; a.r = lowrank; a.dT = deltaT; a.dL = deltaL;
  a.ddT = d_deltaT; a.ddL = d_deltaL; a.dBT = d_BT; a.dBL = d_BL; a.dC = d_C; a.dx = dx;
  a.Wp = Wp; a.wTp = wTp; a.wLp = wLp;
  a.dz = reinterpret_cast<float*>(ws + g.off_dz);
  a.part = reinterpret_cast<float*>(ws + g.off_part);
  a.dWx = d_x_proj_w; a.dwT = d_dt_projT_w; a.dbT = d_dt_projT_b; a.dwL = d_dt_projL_w; a.dbL = d_dt_projL_b;
  const bool f32 = desc->dtype == M2D_F32;
  const size_t lds_data = (size_t)(2 * kTP * kXS + kTP * (g.O + 1)) * 4;
  if (f32) hipLaunchKernelGGL(m2d_proj_bwd_data_kernel<float>, dim3(g.ntiles), dim3(kThreads), lds_data, st, a);
  else hipLaunchKernelGGL(m2d_proj_bwd_data_kernel<bf16_t>, dim3(g.ntiles), dim3(kThreads), lds_data, st, a);
  if (!launched()) return M2D_ERR_HIP;
  const int O4 = (g.O + 3) & ~3;
  const size_t lds_w = (size_t)(kTP * kXS4 + 2 * kTP * kXS + kTP * O4 + kTP * (2 * g.R + 1)) * 4;
  if (!(f32 ? allow_lds_weights<float>() : allow_lds_weights<bf16_t>())) return M2D_ERR_HIP;
  if (f32) hipLaunchKernelGGL(m2d_proj_bwd_weights_kernel<float>, dim3(g.G, g.ne), dim3(kThreads), lds_w, st, a);
  else hipLaunchKernelGGL(m2d_proj_bwd_weights_kernel<bf16_t>, dim3(g.G, g.ne), dim3(kThreads), lds_w, st, a);
  if (!launched()) return M2D_ERR_HIP;
  const int nout = (g.O + 2 * g.R + 2) * g.E;
  hipLaunchKernelGGL(m2d_proj_reduce_kernel, dim3((nout + 255) / 256), dim3(256), 0, st, a);
  return launched() ? M2D_OK : M2D_ERR_HIP;
}

}  // extern "C"

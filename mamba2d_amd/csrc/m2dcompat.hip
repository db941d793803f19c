// m2dcompat: the reference's two native entry points at their own boundary, for gfx950.
//
//   wf_fwd(hs, x, deltaT, deltaL, BT, BL, AT, AL)                         models/kernels/wf_cuda/wf_cuda_bind.cpp:24-33
//   wf_bwd(hs, x, deltaT, deltaL, AT, AL, grad_output, dDAT, dDAL, omega)  models/kernels/wf_cuda/wf_cuda_bind.cpp:35-46
//
// These materialise the (B,H,W,E,N) state tensor, which the fused scan (m2dscan.hip) never does, and they are not
// on the fast path: they exist for callers of the reference's own custom operators (mamba2d::wf_fwd,
// mamba2d::wf_bwd, wavefront_cuda.py:25-57), for any number of states N and for the three element types the
// reference dispatches (wf_cuda.cu:182,240: f64, f32, bf16).  Arithmetic is fp32 for bf16 tensors (each stored
// value is rounded once, where the reference rounds every intermediate) and fp64 for f64.
//
// The reference launches one kernel per anti-diagonal (wf_cuda.cu:187-216, 244-274).  Here a pass is one launch:
// a workgroup owns one image and a chunk of channels with all their states, and walks the diagonals itself; what a
// diagonal needs of the one before was written by the same workgroup, so a workgroup barrier orders it.
#include <hip/hip_runtime.h>

#include <stdint.h>

#include "../../include/m2dscan.h"

namespace {

struct bf16c_t { uint16_t v; };
template <typename T> struct Acc { typedef float type; };
template <> struct Acc<double> { typedef double type; };

template <typename T> __device__ __forceinline__ typename Acc<T>::type ldc(const T* p) { return *p; }
template <> __device__ __forceinline__ float ldc<bf16c_t>(const bf16c_t* p) { return __uint_as_float((uint32_t)p->v << 16); }
template <typename T> __device__ __forceinline__ void stc(T* p, typename Acc<T>::type v) { *p = v; }
template <> __device__ __forceinline__ void stc<bf16c_t>(bf16c_t* p, float v) { p->v = __builtin_bit_cast(uint16_t, (__bf16)v); }
__device__ __forceinline__ float expc(float v) { return __expf(v); }
__device__ __forceinline__ double expc(double v) { return exp(v); }

constexpr int kThreads = 256;

struct WfArgs {
  int B, H, W, E, N;
  int ec;            // channels per workgroup
  int groups;        // workgroups per image
};

// Forward (wf_cuda.cu:40-69): hs[b,i,j,e,n] from hs[b,i-1,j,e,n] and hs[b,i,j-1,e,n], diagonal by diagonal.
template <typename T>
__global__ __launch_bounds__(kThreads) void m2d_wf_fwd_kernel(const WfArgs a, T* hs, const T* x, const T* dT, const T* dL, const T* BT,
                                                              const T* BL, const T* AT, const T* AL) {
  typedef typename Acc<T>::type R;
  const int b = blockIdx.x / a.groups, e0 = (blockIdx.x % a.groups) * a.ec;
  const int ne = a.E - e0 < a.ec ? a.E - e0 : a.ec;      // channels of this workgroup
  const int per_cell = ne * a.N;
  for (int d = 0; d <= a.H + a.W - 2; ++d) {
    const int i_lo = d - (a.W - 1) > 0 ? d - (a.W - 1) : 0, i_hi = d < a.H - 1 ? d : a.H - 1;
    const int work = (i_hi - i_lo + 1) * per_cell;
    for (int idx = threadIdx.x; idx < work; idx += kThreads) {
      const int t = idx / per_cell, rem = idx - t * per_cell;
      const int e = e0 + rem / a.N, n = rem % a.N;
      const int i = i_lo + t, j = d - i;
      const int64_t cell = ((int64_t)b * a.H + i) * a.W + j;
      const R vdT = ldc(dT + cell * a.E + e), vdL = ldc(dL + cell * a.E + e), vx = ldc(x + cell * a.E + e);
      const R uT = vdT * ldc(BT + cell * a.N + n) * vx, uL = vdL * ldc(BL + cell * a.N + n) * vx;
      R h;
      if (i == 0 && j == 0) {
        h = uL;                                                          // the origin takes the L input only (cu:58-59)
      } else if (i == 0) {
        h = expc(vdL * ldc(AL + e * a.N + n)) * ldc(hs + ((cell - 1) * a.E + e) * a.N + n) + uL;
      } else if (j == 0) {
        h = expc(vdT * ldc(AT + e * a.N + n)) * ldc(hs + ((cell - a.W) * a.E + e) * a.N + n) + uT;
      } else {                                                            // sum order as written (cu:65-68)
        const R left = expc(vdL * ldc(AL + e * a.N + n)) * ldc(hs + ((cell - 1) * a.E + e) * a.N + n) + uL;
        const R top = expc(vdT * ldc(AT + e * a.N + n)) * ldc(hs + ((cell - a.W) * a.E + e) * a.N + n) + uT;
        h = (R)0.5 * (left + top);
      }
      stc(hs + (cell * a.E + e) * a.N + n, h);
    }
    __syncthreads();   // the diagonal is in memory before the next one reads it
  }
}

// Backward (wf_cuda.cu:108-160): omega and dBX of a cell from those of its right and lower neighbours, diagonals
// descending; grad_output is overwritten in place by dBX; omega is the reference's two-slot buffer indexed by row.
template <typename T>
__global__ __launch_bounds__(kThreads) void m2d_wf_bwd_kernel(const WfArgs a, const T* hs, const T* dT, const T* dL, const T* AT,
                                                              const T* AL, T* go, T* dDAT, T* dDAL, T* omega) {
  typedef typename Acc<T>::type R;
  const int b = blockIdx.x / a.groups, e0 = (blockIdx.x % a.groups) * a.ec;
  const int ne = a.E - e0 < a.ec ? a.E - e0 : a.ec;
  const int per_cell = ne * a.N;
  const int64_t slot = (int64_t)a.B * a.H * a.E * a.N;   // elements of one omega slot
  for (int d = a.H + a.W - 2; d >= 0; --d) {
    const int i_lo = d - (a.W - 1) > 0 ? d - (a.W - 1) : 0, i_hi = d < a.H - 1 ? d : a.H - 1;
    const int work = (i_hi - i_lo + 1) * per_cell;
    T* om_cur = omega + (d & 1) * slot;
    const T* om_next = omega + ((d + 1) & 1) * slot;
    for (int idx = threadIdx.x; idx < work; idx += kThreads) {
      const int t = idx / per_cell, rem = idx - t * per_cell;
      const int e = e0 + rem / a.N, n = rem % a.N;
      const int i = i_lo + t, j = d - i;
      const int64_t cell = ((int64_t)b * a.H + i) * a.W + j;
      const int64_t at = (cell * a.E + e) * a.N + n;
      const int64_t orow = (((int64_t)b * a.H + i) * a.E + e) * a.N + n;       // omega[.][b][i][e][n]
      const R g = ldc(go + at);
      const bool last_row = i == a.H - 1, last_col = j == a.W - 1;
      R s = g, q = g;
      if (!last_col) {                                                          // right neighbour (i, j+1)
        const R gL = expc(ldc(dL + (cell + 1) * a.E + e) * ldc(AL + e * a.N + n));
        const R mL = (!last_row && i == 0) ? (R)2 : (R)1;                       // (cu:141-146: doubled on the first row, interior case only)
        q += gL * ldc(go + at + (int64_t)a.E * a.N);
        s += mL * gL * ldc(om_next + orow);
      }
      if (!last_row) {                                                          // lower neighbour (i+1, j)
        const R gT = expc(ldc(dT + (cell + a.W) * a.E + e) * ldc(AT + e * a.N + n));
        const R mT = (!last_col && j == 0) ? (R)2 : (R)1;
        q += gT * ldc(go + at + (int64_t)a.W * a.E * a.N);
        s += mT * gT * ldc(om_next + orow + (int64_t)a.E * a.N);
      }
      const R om = (R)0.5 * s;
      stc(om_cur + orow, om);
      stc(go + at, (i > 0 && j > 0) ? (R)0.5 * q : q);                          // dBX (cu:149-152)
      stc(dDAT + at, i > 0 ? (j == 0 ? (R)2 : (R)1) * om * ldc(hs + at - (int64_t)a.W * a.E * a.N) : (R)0);   // (cu:156-157)
      stc(dDAL + at, j > 0 ? (i == 0 ? (R)2 : (R)1) * om * ldc(hs + at - (int64_t)a.E * a.N) : (R)0);         // (cu:159-160)
    }
    __syncthreads();
  }
}

int check(int B, int H, int W, int E, int N, int dtype) {
  if (B < 1 || H < 1 || W < 1 || E < 1 || N < 1) return M2D_ERR_BAD_SHAPE;
  if (dtype != M2D_F32 && dtype != M2D_BF16 && dtype != M2D_F64) return M2D_ERR_UNSUPPORTED;
  return M2D_OK;
}

WfArgs plan(int B, int H, int W, int E, int N) {
  WfArgs a{B, H, W, E, N, 1, 1};
  a.ec = kThreads / N > 0 ? kThreads / N : 1;   // a diagonal cell of a workgroup is about one pass of its threads
  if (a.ec > E) a.ec = E;
  a.groups = (E + a.ec - 1) / a.ec;
  return a;
}

}  // namespace

extern "C" {

int m2d_wf_fwd(int B, int H, int W, int E, int N, int dtype, void* hs, const void* x, const void* deltaT, const void* deltaL,
               const void* BT, const void* BL, const void* AT, const void* AL, void* stream) {
  const int rc = check(B, H, W, E, N, dtype);
  if (rc) return rc;
  const void* req[] = {hs, x, deltaT, deltaL, BT, BL, AT, AL};
  for (const void* q : req) if (!q) return M2D_ERR_NULL_POINTER;
  const WfArgs a = plan(B, H, W, E, N);
  if ((int64_t)B * a.groups >= ((int64_t)1 << 31)) return M2D_ERR_UNSUPPORTED;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)(B * a.groups)), block(kThreads);
  if (dtype == M2D_F32)
    hipLaunchKernelGGL(m2d_wf_fwd_kernel<float>, grid, block, 0, st, a, static_cast<float*>(hs), static_cast<const float*>(x), static_cast<const float*>(deltaT),
                       static_cast<const float*>(deltaL), static_cast<const float*>(BT), static_cast<const float*>(BL), static_cast<const float*>(AT), static_cast<const float*>(AL));
  else if (dtype == M2D_F64)
    hipLaunchKernelGGL(m2d_wf_fwd_kernel<double>, grid, block, 0, st, a, static_cast<double*>(hs), static_cast<const double*>(x), static_cast<const double*>(deltaT),
                       static_cast<const double*>(deltaL), static_cast<const double*>(BT), static_cast<const double*>(BL), static_cast<const double*>(AT), static_cast<const double*>(AL));
  else
    hipLaunchKernelGGL(m2d_wf_fwd_kernel<bf16c_t>, grid, block, 0, st, a, static_cast<bf16c_t*>(hs), static_cast<const bf16c_t*>(x), static_cast<const bf16c_t*>(deltaT),
                       static_cast<const bf16c_t*>(deltaL), static_cast<const bf16c_t*>(BT), static_cast<const bf16c_t*>(BL), static_cast<const bf16c_t*>(AT), static_cast<const bf16c_t*>(AL));
  return hipGetLastError() == hipSuccess ? M2D_OK : M2D_ERR_HIP;
}

int m2d_wf_bwd(int B, int H, int W, int E, int N, int dtype, const void* hs, const void* x, const void* deltaT, const void* deltaL,
               const void* AT, const void* AL, void* grad_output, void* dDAT, void* dDAL, void* omega, void* stream) {
  const int rc = check(B, H, W, E, N, dtype);
  if (rc) return rc;
  (void)x;   // (unused by the reference's kernel as well, wf_cuda.cu:76)
  const void* req[] = {hs, deltaT, deltaL, AT, AL, grad_output, dDAT, dDAL, omega};
  for (const void* q : req) if (!q) return M2D_ERR_NULL_POINTER;
  const WfArgs a = plan(B, H, W, E, N);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)(B * a.groups)), block(kThreads);
  if (dtype == M2D_F32)
    hipLaunchKernelGGL(m2d_wf_bwd_kernel<float>, grid, block, 0, st, a, static_cast<const float*>(hs), static_cast<const float*>(deltaT), static_cast<const float*>(deltaL),
                       static_cast<const float*>(AT), static_cast<const float*>(AL), static_cast<float*>(grad_output), static_cast<float*>(dDAT), static_cast<float*>(dDAL), static_cast<float*>(omega));
  else if (dtype == M2D_F64)
    hipLaunchKernelGGL(m2d_wf_bwd_kernel<double>, grid, block, 0, st, a, static_cast<const double*>(hs), static_cast<const double*>(deltaT), static_cast<const double*>(deltaL),
                       static_cast<const double*>(AT), static_cast<const double*>(AL), static_cast<double*>(grad_output), static_cast<double*>(dDAT), static_cast<double*>(dDAL), static_cast<double*>(omega));
  else
    hipLaunchKernelGGL(m2d_wf_bwd_kernel<bf16c_t>, grid, block, 0, st, a, static_cast<const bf16c_t*>(hs), static_cast<const bf16c_t*>(deltaT), static_cast<const bf16c_t*>(deltaL),
                       static_cast<const bf16c_t*>(AT), static_cast<const bf16c_t*>(AL), static_cast<bf16c_t*>(grad_output), static_cast<bf16c_t*>(dDAT), static_cast<bf16c_t*>(dDAL), static_cast<bf16c_t*>(omega));
  return hipGetLastError() == hipSuccess ? M2D_OK : M2D_ERR_HIP;
}

}  // extern "C"

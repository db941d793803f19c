// m2dscan: wavefront 2-D selective scan for gfx950 (MI355X), forward and backward.
//
// The recurrence (reference: models/kernels/wf_cuda/wf_cuda.cu:40-69)
//     h[i,j] = cL*(aL*h[i,j-1] + uL) + cT*(aT*h[i-1,j] + uT),   a = exp(delta*A),  u = delta*B*x
// with (cT,cL) = (0,1) on the first row, (1,0) on the first column and (1/2,1/2) inside, is
// independent across (batch, channel, state).
//
// Mapping.  The grid rows are cut in bands of 14 rows.  A 64-lane wavefront owns 4 channel slots
// of one image: lane = slot*16 + r, where lanes r = 1..14 hold band rows, lane 0 a ghost of the
// row above the band and lane 15 (backward only) a ghost of the row below it.  Every lane walks a
// "stream" of positions: position s = (band, column) = (s / S, s % S) with a stride S >= W, and at
// global step t lane r is at position t - r, so one step of the wave is an anti-diagonal of a
// band for 4 channels at once, and when S = W a lane enters column 0 of the next band on the step
// after it left the last column of the current one: the pipeline never drains between bands.
// The 16 states of the cell stay in VGPRs; h[i,j-1] is the lane's own previous value, h[i-1,j] is
// the previous value of the lane below, fetched with a DPP row shift; the first row of a band
// takes it from the ghost lane, which replays the last row of the band above out of a small
// buffer in memory.  y = C.h is a 16-term sum in registers.
//
// The factor 1/2 and the first-row/column cases are folded into the gate exponent
// (exp2(delta*A*log2e + log2 c)) and into the input coefficient: the inner loop is branch-free,
// and lanes are never masked (rows and cells outside the grid work on zero operands).
//
// Backward (adjoint; reference wf_cuda.cu:108-160 and models/kernels/wavefront_cuda.py:97-139,
// 176-178, 193-194).  The forward stores the register state every CK steps (one anti-diagonal
// per checkpoint).  The backward walks the steps in reverse, a block of CK at a time: restore the
// checkpoint, recompute the CK states into registers, then run the adjoint over the block
// backwards,
//     lambda = dy*C + muL(own, previous step) + muT(lane above, previous step)
//     muT = cT*aT*lambda,  muL = cL*aL*lambda
// emitting every gradient on the fly.  Channel sums (d_BT, d_BL, d_C) are reduced inside the
// wave with lane-swap butterflies over the channel slots, then across the 8 waves of the
// workgroup through LDS in a fixed order, then across workgroups by a small kernel.  Sums over
// positions (d_AT, d_AL, d_D) are register accumulators reduced at the end.  No atomics:
// results are bit-reproducible.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdio>
#include <cstring>
#include <stdint.h>
#include <type_traits>

#include "../../include/m2dscan.h"

// Scratch of m2d_scan_fwd_noalloc: the workspace of a forward call, for callers that cannot
// allocate.  Every device that loads the library holds its own copy at its own address; host code
// only ever uses the address that hipGetSymbolAddress returns for the current device.
static __device__ __align__(256) unsigned char scratch[M2D_NOALLOC_SCRATCH_BYTES];

namespace {

constexpr int kN = 16;            // states per channel
#ifndef M2D_CK
#define M2D_CK 4
#endif
constexpr int kCK = M2D_CK;       // checkpoint interval (steps)
constexpr int kHB = 16;           // rows per band = lanes per DPP row
constexpr int kHBShift = 4;
constexpr int kRB = 14;           // grid rows per band; lanes 0 and 15 of a row are boundary ghosts
constexpr int kFwdWaves = 8;      // waves per forward workgroup
constexpr int kFwdHalfWaves = 4;  // ... of a small batch (fewer workgroups of 8 than half the compute units)
constexpr int kBwdWaves = 8;      // waves per backward workgroup
constexpr int kZeroFloats = 64;     // page of zeros at the head of the set-up area
constexpr int kModeSweep = 0, kModeSliced = 1, kModeStacked = 2;   // how the bands of the batch are scheduled
constexpr int kLinkLag = 7;        // linked sweep: blocks by which a band trails the band it depends on (see link_need_*)
constexpr int kSpinLimit = 1 << 21;   // linked sweep: polls of a neighbour's progress before a workgroup gives up waiting
// Words from one progress count of the linked sweep to the next: a count has 256 bytes to itself.  Side by side in one
// cache line, the counts of a band's workgroups were written by 16 workgroups while 64 waves polled the line, and
// every hand-off waited for that line (256x256, E=64: forward 0.46 -> 0.34 ms with the counts apart).
constexpr int kLinkStride = 64;
constexpr uint32_t kLinkAbort = 0xffffffffu;   // progress value of a band that gave up: nobody waits for it
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

struct bf16_t { uint16_t v; };
typedef float v4f_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) v4f_t lds_float4;   // a float4 known to live in LDS

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t lo16) { return __uint_as_float(lo16 << 16); }
// round to nearest even; one instruction on gfx950 (v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }

template <typename T> struct IO;
template <> struct IO<float> {
  static __device__ __forceinline__ float ld(const float* p) { return *p; }
  static __device__ __forceinline__ void st(float* p, float v) { *p = v; }
  template <int EC> static __device__ __forceinline__ void ldv(const float* p, float (&v)[EC]) {
    if constexpr (EC == 2) { float2 t = *reinterpret_cast<const float2*>(p); v[0] = t.x; v[1] = t.y; }
    else { for (int c = 0; c < EC; ++c) v[c] = p[c]; }
  }
  template <int EC> static __device__ __forceinline__ void stv(float* p, const float (&v)[EC]) {
    if constexpr (EC == 2) { *reinterpret_cast<float2*>(p) = make_float2(v[0], v[1]); }
    else { for (int c = 0; c < EC; ++c) p[c] = v[c]; }
  }
  static __device__ __forceinline__ void st4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
};
template <> struct IO<bf16_t> {
  static __device__ __forceinline__ float ld(const bf16_t* p) { return bf16_bits_to_f32(p->v); }
  static __device__ __forceinline__ void st(bf16_t* p, float v) { p->v = f32_to_bf16_bits(v); }
  template <int EC> static __device__ __forceinline__ void ldv(const bf16_t* p, float (&v)[EC]) {
    if constexpr (EC == 2) {
      uint32_t t = *reinterpret_cast<const uint32_t*>(p);
      v[0] = __uint_as_float(t << 16); v[1] = __uint_as_float(t & 0xffff0000u);
    } else { for (int c = 0; c < EC; ++c) v[c] = bf16_bits_to_f32(p[c].v); }
  }
  template <int EC> static __device__ __forceinline__ void stv(bf16_t* p, const float (&v)[EC]) {
    if constexpr (EC == 2) {
      *reinterpret_cast<uint32_t*>(p) = (uint32_t)f32_to_bf16_bits(v[0]) | ((uint32_t)f32_to_bf16_bits(v[1]) << 16);
    } else { for (int c = 0; c < EC; ++c) p[c].v = f32_to_bf16_bits(v[c]); }
  }
  static __device__ __forceinline__ void st4(bf16_t* p, float4 v) {
    uint2 t;
    t.x = (uint32_t)f32_to_bf16_bits(v.x) | ((uint32_t)f32_to_bf16_bits(v.y) << 16);
    t.y = (uint32_t)f32_to_bf16_bits(v.z) | ((uint32_t)f32_to_bf16_bits(v.w) << 16);
    *reinterpret_cast<uint2*>(p) = t;
  }
};

__device__ __forceinline__ void ld16f(const float* p, float (&v)[kN]) {
  const float4* q = reinterpret_cast<const float4*>(p);
#pragma unroll
  for (int k = 0; k < 4; ++k) { float4 t = q[k]; v[4*k] = t.x; v[4*k+1] = t.y; v[4*k+2] = t.z; v[4*k+3] = t.w; }
}

// Rows of 16 lanes (one band of one channel slot).  Lane r receives the value of lane r-1 of
// its row (lane 0, which has no lane below, receives 0) ...
__device__ __forceinline__ float from_row_below(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x111 /*row_shr:1*/, 0xf, 0xf, true));
}
// The same move folded into the instruction that uses the value (the compiler does this for adds
// but not for multiply-adds): acc + a * (v of the lane below), a * (v of the lane below),
// a + (v of the lane above).  The operand v is always a value of the step before, produced many
// instructions earlier, so the two wait states a DPP read needs after a VALU write of the same
// register have long passed.
__device__ __forceinline__ float fma_row_below(float a, float v, float acc) {
  asm("v_fmac_f32_dpp %0, %1, %2 row_shr:1 row_mask:0xf bank_mask:0xf bound_ctrl:1" : "+v"(acc) : "v"(v), "v"(a));
  return acc;
}
__device__ __forceinline__ float mul_row_below(float a, float v) {
  float d;
  asm("v_mul_f32_dpp %0, %1, %2 row_shr:1 row_mask:0xf bank_mask:0xf bound_ctrl:1" : "=v"(d) : "v"(v), "v"(a));
  return d;
}
__device__ __forceinline__ float add_row_above(float a, float v) {
  float d;
  asm("v_add_f32_dpp %0, %1, %2 row_shl:1 row_mask:0xf bank_mask:0xf bound_ctrl:1" : "=v"(d) : "v"(v), "v"(a));
  return d;
}
// ... or the value of lane r+1 (lane 15 receives 0).
__device__ __forceinline__ float from_row_above(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x101 /*row_shl:1*/, 0xf, 0xf, true));
}
__device__ __forceinline__ float fexp2(float v) { return __builtin_amdgcn_exp2f(v); }

// d softplus(z) / dz from the softplus value d: sigmoid(z) = 1 - exp(-d).  For fp32 tensors small
// values take the series, where the difference would cancel; for bf16 tensors the cancellation
// (relative error 1e-3 at d = 1e-4) stays below the rounding of the result.
template <typename T>
__device__ __forceinline__ float softplus_slope(float d) {
  const float direct = 1.f - fexp2(-kLog2e * d);
  if constexpr (sizeof(T) == 2) return direct;
  const float series = d * __builtin_fmaf(d, __builtin_fmaf(d, __builtin_fmaf(d, -1.f / 24.f, 1.f / 6.f), -0.5f), 1.f);
  return d < 0.0625f ? series : direct;
}
// All four values exist from here on: nothing may compute one of them later, next to its use.
// (An empty statement; with the scheduling barrier behind it, it keeps a group of v_exp_f32 in
// front of the instructions that follow the barrier.)
__device__ __forceinline__ void pin4(float (&a)[4]) { asm volatile("" : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3])); }

// a[lanes 32..63] <-> b[lanes 0..31]; returns a+b: lanes 0..31 hold the two-half sum of a,
// lanes 32..63 that of b.
__device__ __forceinline__ float fold32(float a, float b) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(b), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
// rows of 16 lanes: a.row1 <-> b.row0, a.row3 <-> b.row2; returns a+b: even rows hold the
// (row, row+1) sum of a, odd rows that of b.
__device__ __forceinline__ float fold16(float a, float b) {
  auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

struct ScanParams {
  const void *x, *dT, *dL, *dy;
  const float *bt, *bl, *cc;        // B_T, B_L, C in fp32, state n of a cell at [cell*bc_stride + spos(n)]
  const float *A2T, *A2L, *Df;      // A*log2(e) and D in fp32, (E,16) / (E)
  const float* zeros;               // 256 bytes of zeros (source for out-of-grid staging chunks)
  void *y, *dx, *ddT, *ddL;
  float* ckpt;                      // [B][ck_nblk][E][2][16][2][4]  state snapshots, one per kept block of steps: quad q of lane row r (see snap_quad) holds the states sinv(4q .. 4q+3); bf16 for 16-bit tensors
  float* top;                       // [nbands-1][B][W][E][16]       last row of each band (forward states)
  float* bot;                       // [nbands or 1][B][W][E][16]    first-row muT of a band, for the band above (adjoint)
  float* part;                      // [G][P][3][16]                 per-workgroup channel sums of d_C, d_BT, d_BL
  float* pA;                        // [B*pa_slots][E][2][16]
  float* pD;                        // [B*pa_slots][E]
  int B, H, W, E;
  int nbands, nblk, bc_stride, flip;
  int bc_direct;                    // forward without snapshots: B_T, B_L, C are staged from the caller's tensors (states in natural order)
  const void* bcd[4];               // ... those tensors (B_T, B_L, C; the fourth entry pads)
  int dpre;                         // backward: d_deltaT, d_deltaL leave multiplied by the slope of the softplus that made the deltas
  int S;                            // stream stride: positions per band (>= W)
  int T_total;                      // steps of the whole sweep
  int rows_last;                    // grid rows of the last band
  int rb;                           // grid rows of every other band: 14 (kRB), or for stacked images the largest multiple of the image height up to 16
  uint32_t magicS;                  // floor(2^32 / S)
  // Linked sweep (few images, many bands): every band has its own workgroups, all in one launch; a
  // band publishes how many blocks of its window are done (boundary rows in memory) and the band
  // that reads its boundary rows polls that count before it stages them.
  int sliced;                       // on/off
  int sl_nbb;                       // blocks per band (S / kCK)
  uint32_t* prog;                   // [nbands][B][workgroups per image] blocks of the band's window whose boundary rows are in memory
  uint32_t* link_err;               // set to 1 by a workgroup that gave up waiting (results are then invalid)
  int link_test;                    // test aid (M2D_FLAG_TEST_DEAD_LINK): 1 + the band whose neighbour never reports, and a wait gives up after a few polls
  int64_t bot_stride;               // floats between the mu_T rows of consecutive bands (0: one row buffer, bands in sequence)
  int pa_slots;                     // partial sums over positions per image (1, or one per band when sliced)
  // Stacked images (grids of at most 16 rows, one band each): `ips` images in a row of the batch
  // are swept as one tall image whose bands do not depend on each other: B, H above are then the
  // number and height of the stacks, and a workgroup shortens H for a last, shorter stack.
  int stacked, ips, Himg, Breal;    // on/off, images per stack, rows per image, images in the batch
  int Hs;                           // rows between the bases of consecutive (stacked) images
  int64_t Ptot;                     // cells of the whole batch
  int bpb;                          // workgroups per image
  int nwg;                          // total workgroups
  // Checkpoint interval: the forward keeps the snapshot of one block in 2^ck_shift (the first of every such group
  // of a workgroup's window); the backward replays the forward over the other blocks of a group before it sweeps
  // the group, and parks their snapshots in `ring`.
  int ck_shift;
  int ck_half;                      // a snapshot every 2 steps (before the steps 0 and 2 of every block, and one behind the last block): snapshot 2m + s is the state before step 4m + 2s
  int ck_pb;                        // kept snapshots per band (linked sweep)
  int ck_nblk;                      // kept snapshots per image
  void* ring;                       // [workgroup][2^ck_shift - 1][channel of the workgroup][4][16] snapshot quads
};

// Workgroups are dealt round-robin to the 8 XCDs; renumber so that consecutive logical ids
// (the channel groups of one image, which share B, C and cache lines of x) sit on one XCD and
// therefore share its L2.
__device__ __forceinline__ int logical_block(int nwg) {
  const int id = blockIdx.x;
  const int per = nwg >> 3;
  if (per == 0 || id >= (per << 3)) return id;
  return (id & 7) * per + (id >> 3);
}

// Stream position -> (band, column).  s >= -21 (S >= 7, so 3 strides below zero are in range).
// Bands outside [0, nbands) and columns >= W are not on the grid.
struct Pos { int bnd, col; };
__device__ __forceinline__ Pos pos_of(const ScanParams& p, int s) {
  const uint32_t sp = (uint32_t)(s + 3 * p.S);
  uint32_t q = __umulhi(sp, p.magicS);          // q or q-1 of the true quotient for sp < 2^32
  uint32_t rem = sp - q * (uint32_t)p.S;
  if (rem >= (uint32_t)p.S) { q += 1; rem -= (uint32_t)p.S; }
  Pos o; o.bnd = (int)q - 3; o.col = (int)rem;
  return o;
}
__device__ __forceinline__ int band_rows(const ScanParams& p, int bnd) { return bnd == p.nbands - 1 ? p.rows_last : p.rb; }
// Row of its band that lane row r works on: lanes 1 .. 14 the rows 0 .. 13, lane 0 (-1) and lane 15 the ghosts of the
// rows next to the band.  The bands of stacked images have no neighbours to replay: all 16 lanes are rows there.
__device__ __forceinline__ int grid_row(const ScanParams& p, int r) { return p.stacked ? r : r - 1; }
// cell index inside its image of lane row r of band bnd at column col
__device__ __forceinline__ int cell_of(const ScanParams& p, int bnd, int r, int col) {
  const int cell = __mul24(bnd * p.rb + grid_row(p, r), p.W) + col;   // rows and columns are far below 2^24
  return p.flip ? p.H * p.W - 1 - cell : cell;
}

// Position of state n inside a 16-float record.  With PERM the four states that the backward
// folds together (n = q*4 + m for q = 0..3) sit in one float4, in fold order.
template <bool PERM> __device__ __forceinline__ constexpr int spos(int n) {
  if (!PERM) return n;
  const int q = n >> 2, m = n & 3;
  return 4 * m + ((q == 1) ? 2 : (q == 2) ? 1 : q);
}

// state stored at position pos of a record (inverse of spos)
template <bool PERM> __device__ __forceinline__ constexpr int sinv(int pos) {
  if (!PERM) return pos;
  const int m = pos >> 2, qi = pos & 3;
  return ((qi == 1) ? 2 : (qi == 2) ? 1 : qi) * 4 + m;
}

// ------------------------------------------------------------------------------ operand staging
// The operands of a block of kCK steps of a band are copied to LDS one block ahead of their use
// with direct global->LDS loads (no registers, asynchronous): lane i of a wave-wide copy fills
// the 16-byte chunk i of a 1 KB LDS window.  Every copy is laid out so that the chunk a lane fills
// belongs to the lane's own row (lane & 15): the position arithmetic of a block is done once per
// lane and serves the lane's copies and its own loads and stores alike.  One buffer, in planes of
// 256 bytes (16 chunks):
//   per step k, kPlanes planes:
//     planes 0..11   BC : plane 4*tensor + g holds, for the 16 lane rows r, the four values of state
//                         group g of B_T, B_L, C (tensor 0, 1, 2) of the cell (row r, column t0+k-r);
//     planes 12..    TOP: plane 12 + 4*h + g holds, for the channels 16h..16h+15 of the workgroup, state
//                         group g of the last row of the band above at column t0+k;
//     then (adjoint) BOT: the same for the muT of the first row of the band below at column t0+k-15;
//     then           K  : chunk r holds the gate offsets and input coefficients of lane row r at this step;
//   then XD: per tensor (x, deltaT, deltaL[, dy]), step k and chunk of channels, the 16 lane rows side by
//        side (chunk index = ((tensor*kCK + k)*kCpt + channel chunk)*16 + r); needs E to be a multiple
//        of a chunk.
// A grid row reads the groups of its B_T, B_L, C at r*16 plus plane offsets; the upper ghost (lane 0)
// reads the TOP planes of its channel as its B_T, the lower ghost (lane 15) the BOT planes as its C:
// a per-lane base address under the same immediate offsets.  Chunks of rows and cells outside the grid
// are filled from a page of zeros: such lanes compute on finite operands and never need to be masked.
template <typename T, int NT, int CW, bool WITH_BOT>
struct Stage {
  static constexpr int kElem = 16 / sizeof(T);           // elements per chunk
  static constexpr int kCpt = CW >= kElem ? CW / kElem : 1;   // chunks per tensor per cell (fewer channels than a chunk: the chunk they are in)
  static constexpr int kXStepBytes = kCpt * kHB * 16;    // XD bytes per tensor and step
  static constexpr int kXTauBytes = kCK * kXStepBytes;   // XD bytes per tensor
  static constexpr int kXTauInstr = kXTauBytes / 1024;   // wave-wide copies per tensor
  static constexpr int kPlane = kHB * 16;                // bytes per plane
  static constexpr int kG16 = (CW + 15) / 16;            // groups of 16 channels (a workgroup of fewer copies the rows of 16 all the same)
  static constexpr int kTopPlane = 12;
  static constexpr int kBotPlane = kTopPlane + 4 * kG16;
  // (adjoint: at least 24 planes, so that what a ghost reads 4 and 8 planes behind its boundary row is inside the step)
  static constexpr int kPlanes = WITH_BOT ? (kTopPlane + 8 * kG16 > 24 ? kTopPlane + 8 * kG16 : 24) : kTopPlane + 4 * kG16;
  static constexpr int kConstPlane = kPlanes;            // plane of the rows' gate and input constants at this step
  static constexpr int kKStr = (kPlanes + 1) * kPlane;   // bytes per step
  static constexpr int kBLOff = 4 * kPlane, kCOff = 8 * kPlane;   // B_L and C planes behind the B_T planes
  static constexpr int kXOff = kCK * kKStr;
  static constexpr int kBytes = kXOff + NT * kXTauBytes; // one buffer
  static_assert(kXTauBytes % 1024 == 0, "a wave-wide copy must not straddle two tensors of XD");
  static_assert(kCpt <= 2 || kCpt % 4 == 0, "a wave-wide copy of XD covers one step, or two halves of 32 lanes (one chunk per cell: XD is not staged)");
  static_assert(CW % kElem == 0 || kElem % CW == 0, "a workgroup's channels fill whole chunks, or one part of a chunk");
  static_assert(CW % 16 == 0 || CW < 16, "boundary rows are copied 16 channels at a time");
  // byte offset inside a tensor's part of XD of channel `ch` (of the workgroup) for lane row r at step 0
  static __host__ __device__ constexpr uint32_t x_off(int r, int ch) {
    return (uint32_t)(((ch / kElem) * kHB + r) * 16 + (ch % kElem) * (int)sizeof(T));
  }
  // where the ghost of channel `ch` finds group 0 of the boundary row at step 0
  static __host__ __device__ constexpr uint32_t top_off(int ch) { return (uint32_t)((kTopPlane + 4 * (ch / 16)) * kPlane + (ch % 16) * 16); }
  static __host__ __device__ constexpr uint32_t bot_off(int ch) { return (uint32_t)((kBotPlane + 4 * (ch / 16)) * kPlane + (ch % 16) * 16); }
};

// One wave-wide direct load: lane i copies 16 bytes from its own global address to
// lds_window + 16*i.  Written as inline assembly on purpose: the copy is asynchronous, and its
// completion is awaited once per block by staging_landed() (counter vmcnt), not before every LDS
// read that follows it, which is what the compiler does for the builtin.
// DEVICE_SCOPE: read past the L1 (data written earlier in the same launch by this workgroup).
template <bool DEVICE_SCOPE>
__device__ __forceinline__ void lds_fill16(const void* src, char* lds_window) {
  const uint32_t base = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) char*)lds_window);
  if constexpr (DEVICE_SCOPE)
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off sc1" ::"v"(src), "s"(base) : "memory", "m0");
  else
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(base) : "memory", "m0");
}

// ---- linked sweep: hand-off between the workgroups of neighbouring bands inside one launch.
// Boundary rows and progress counts are written through to memory and read past the caches at
// device scope (sc1), so that workgroups on different XCDs, whose L2 caches are not coherent with
// each other, see them; plain vector loads and stores, no fences.  A workgroup only ever waits for
// a workgroup with a lower index, which was dispatched before it, so the one with the lowest index
// that is not finished is always running: every wait ends.  Should one not (a defect), the waiting
// workgroup gives up after kSpinLimit polls, flags the error and tells its own dependants not to
// wait either, so that the launch still ends.
__device__ __forceinline__ uint32_t link_poll(const uint32_t* ptr) {
  uint32_t v;
  asm volatile("global_load_dword %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(ptr) : "memory");
  return __builtin_amdgcn_readfirstlane(v);
}
__device__ __forceinline__ void link_publish(uint32_t* ptr, uint32_t v) {
  asm volatile("global_store_dword %0, %1, off sc1" ::"v"(ptr), "v"(v) : "memory");
}
// 16 bytes of a boundary row, written through at device scope
__device__ __forceinline__ void store_row_device_scope(float4* dst, float4 v) {
  const v4f_t w = {v.x, v.y, v.z, v.w};
  asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(dst), "v"(w) : "memory");
}
template <int PUB>   // the thread that publishes: one of a wave that waits, so that it knows of a wait given up
struct LinkT {
  uint32_t* mine = nullptr;         // this workgroup's progress count
  const uint32_t* dep = nullptr;    // the count of the workgroup whose boundary rows this one reads (none: first band of the sweep)
  uint32_t seen = 0;                // last value read from dep
  bool gave_up = false;
  uint32_t* err = nullptr;
  int limit = kSpinLimit;           // polls before a wait gives up
  static constexpr int pub = PUB;
  // test aid: the workgroups of band `link_test - 1` wait for a count that nobody publishes (a word of the header,
  // zero for the whole launch), and every wait of the launch gives up after a few polls: the give-up path runs, and
  // every workgroup still ends
  __device__ __forceinline__ void rig(const ScanParams& p, int band) {
    if (p.link_test) {
      limit = 16;
      if (band == p.link_test - 1) dep = p.link_err + 1;
    }
  }
  // this workgroup's results mean nothing: it gave up waiting, or a band it depends on did
  __device__ __forceinline__ bool broken() const { return gave_up || seen == kLinkAbort; }
  // (uniform) returns once the neighbour has `need` blocks done
  __device__ __forceinline__ void wait_for(uint32_t need) {
    if (!dep || seen >= need) return;
    for (int spin = 0; spin < limit; ++spin) {
      seen = link_poll(dep);
      if (seen >= need) return;
      __builtin_amdgcn_s_sleep(4);
    }
    seen = kLinkAbort;
    gave_up = true;
    if ((int)threadIdx.x == pub) link_publish(err, 1u);
  }
  // after a barrier behind which `done` blocks of this band have their boundary rows in memory
  __device__ __forceinline__ void publish(uint32_t done) {
    if ((int)threadIdx.x == pub) link_publish(mine, (gave_up || seen == kLinkAbort) ? kLinkAbort : done);
  }
};
using Link = LinkT<0>;
// Blocks of the neighbour's window that must be done before block j of a band's own window is staged.
// Forward: the ghost of block j replays the columns 4j .. 4j+3 of the last row of the band above,
// which lane 14 stored at the window's steps 4j+14 .. 4j+17, the last of them in block j+4.
// Backward (blocks are swept from the last to the first, counts are blocks done from the end): the lower
// ghost of block j reads the columns 4j-15 .. 4j-12 of the first row of the band below, which lane 1 stored
// at steps 4j-14 .. 4j-11, the earliest of them in block j-4.
__device__ __forceinline__ uint32_t link_need_fwd(int j, int nbb) { return (uint32_t)(j + 5 < nbb ? j + 5 : nbb); }
__device__ __forceinline__ uint32_t link_need_bwd(int j, int nbb) { return (uint32_t)(j - 4 > 0 ? nbb - (j - 4) : nbb); }

// Position of the stream index (index of A) + d, for 0 <= d < 19.  Strides below 19 (stacked
// images) can wrap more than once.
__device__ __forceinline__ Pos pos_after(const ScanParams& p, Pos A, int d) {
  Pos q;
  q.col = A.col + d;
  q.bnd = A.bnd;
  if (q.col >= p.S) { q.col -= p.S; q.bnd += 1; }
  if (p.S < kHB + kCK - 1) {   // uniform
    if (q.col >= p.S) { q.col -= p.S; q.bnd += 1; }
    if (q.col >= p.S) { q.col -= p.S; q.bnd += 1; }
  }
  return q;
}

// Every load the compiler knows about has returned (vmcnt 0, other counters untouched).  Placed
// after the start-up loads so that no conservative wait for them is emitted inside the main
// loop, where it would also wait for the asynchronous staging copies.
__device__ __forceinline__ void settle_loads() { __builtin_amdgcn_s_waitcnt(0x0F70); }

// Two waves share a SIMD where a workgroup has 8 (wave w and wave w + 4), and between two barriers both have the same
// work.  Left alone the instruction arbiter favours the older wave throughout: it reaches the barrier early and
// idles there while the younger one finishes alone, at the rate of a single wave (a quarter of the older waves'
// time went into such waits in the backward kernel).  So the younger wave raises its priority for the first part of
// every barrier interval and drops it for the rest, where age favours the older one again: both arrive together.
// (s_setprio changes the wave's own priority among the waves of its SIMD, nothing else.)
template <int NW>
__device__ __forceinline__ void lead_if_younger(int wave, bool lead) {
  if constexpr (NW == 8) {
    if (wave >= NW / 2) { if (lead) __builtin_amdgcn_s_setprio(1); else __builtin_amdgcn_s_setprio(0); }
  }
}

// all direct-to-LDS loads of this wave have landed ...
__device__ __forceinline__ void staging_landed() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0); known to the compiler, so loads it tracks need no further wait
  asm volatile("" ::: "memory");
}
// The same with the N youngest vector-memory operations of the wave left in flight.  The counter
// retires loads and stores in issue order, so everything older than those N has completed; the
// caller must know that at least N operations were issued after the loads it waits for.
template <int N>
__device__ __forceinline__ void staging_landed_behind() {
  static_assert(N >= 0 && N < 16, "low bits of the counter field only");
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt(0x0F70 | N);
  asm volatile("" ::: "memory");
}
// The same with a count that is only known at run time (uniform; counts above 7 wait as for 7).
__device__ __forceinline__ void staging_landed_behind_n(int n) {
  switch (n < 0 ? 0 : (n > 7 ? 7 : n)) {
    case 0: staging_landed(); break;
    case 1: staging_landed_behind<1>(); break;
    case 2: staging_landed_behind<2>(); break;
    case 3: staging_landed_behind<3>(); break;
    case 4: staging_landed_behind<4>(); break;
    case 5: staging_landed_behind<5>(); break;
    case 6: staging_landed_behind<6>(); break;
    default: staging_landed_behind<7>(); break;
  }
}
// ... and those of the other waves too
__device__ __forceinline__ void staging_fence() {
  staging_landed();
  __syncthreads();
}

// Per-lane constants of the band a lane is in.  Lanes 1..14 of every 16-lane row are grid rows;
// lane 0 is a ghost that replays the last row of the band above (it reads its "B_T" from the TOP
// record with input coefficient 1 and closed gates, so its state IS that row), lane 15 is the
// ghost of the first row of the band below for the adjoint (open T gate with delta 0 and dy = 1 on
// the staged row of mu_T).  All of this is operand selection: the inner loops have no boundary cases.
struct LaneK {
  bool real;                   // a grid row of its band (and a valid channel)
  float oT, oL, cT, cL;        // gate offsets (log2 of the coefficient) and input coefficients inside the grid
  float oT0, cT0, cL0;         // the same at column 0 (the left gate is closed there)
};
template <bool BWD>
__device__ __forceinline__ LaneK lane_consts(const ScanParams& p, int bnd, int r, bool ch_ok) {
  const float ninf = -__builtin_huge_valf();
  // `bnd` is a band of the grid (callers clamp): a row that is before the first band or past the
  // last one works on zero operands with the constants of that band
  LaneK c;
  const int gr = grid_row(p, r);
  c.real = ch_ok && gr >= 0 && gr < band_rows(p, bnd);
  // grid row 0 of an image: no row above (stacked images: a band holds whole images)
  const bool first_row = p.stacked ? gr % p.Himg == 0 : (bnd == 0 && gr == 0);
  const bool gbot = BWD && !p.stacked && r == kHB - 1 && bnd + 1 < p.nbands;
  c.oT = gbot ? 0.f : (!c.real || first_row ? ninf : -1.f);
  c.oL = !c.real ? ninf : (first_row ? 0.f : -1.f);
  c.cT = !c.real || first_row ? 0.f : 0.5f;
  c.cL = !c.real ? 0.f : (first_row ? 1.f : 0.5f);
  c.oT0 = gbot ? 0.f : (!c.real || first_row ? ninf : 0.f);
  c.cT0 = !c.real || first_row ? 0.f : 1.f;
  c.cL0 = c.real && first_row ? 1.f : 0.f;
  return c;
}

// The forward keeps, and the backward restores, the state of a lane at the start of a block only
// if the lane's previous position was a cell of the grid (the ghost: a cell of the row above).
__device__ __forceinline__ bool snapshot_lane(const ScanParams& p, Pos at, int r, bool ch_ok) {
  Pos pv;
  pv.bnd = at.col >= 1 ? at.bnd : at.bnd - 1;
  pv.col = at.col >= 1 ? at.col - 1 : p.S - 1;
  const int gr = grid_row(p, r);
  const bool row_ok = gr < 0 ? pv.bnd >= 1 : gr < band_rows(p, pv.bnd);
  return ch_ok && (unsigned)pv.bnd < (unsigned)p.nbands && pv.col < p.W && row_ok;
}

// Positions of one lane row over a block of kCK steps.  All rows of the wave sit within 19
// consecutive stream positions, which touch at most two bands, so everything derives from the
// (wave-uniform) position A of the stream index t0 - 15 with adds and compares.
struct BlockPos {
  int bnd0, col0;      // position at the first step of the block
  int kw;              // first step of the block at which the row is in the next band (>= kCK: never)
  int kz;              // step of the block at which the row is at column 0 (>= kCK: never)
  uint32_t in_grid;    // bit k: the row is at a cell of the grid at step k
};
// Lane row r is a row of the grid in the bands 0 .. row_bands(r) - 1 (none for a ghost lane; a row
// beyond the height of the last band misses that one).  A lane constant.
__device__ __forceinline__ int row_bands(const ScanParams& p, int r) {
  const int gr = grid_row(p, r);
  return (gr >= 0 && gr < p.rb) ? p.nbands - 1 + (gr < p.rows_last ? 1 : 0) : 0;
}
// bits k < n of a block's steps
__device__ __forceinline__ uint32_t steps_below(int n) { return (1u << (n < 0 ? 0 : (n > kCK ? kCK : n))) - 1u; }
__device__ __forceinline__ BlockPos block_pos(const ScanParams& p, Pos A, int r, int rbands) {
  BlockPos q;
  const Pos at = pos_after(p, A, kHB - 1 - r);
  q.col0 = at.col; q.bnd0 = at.bnd;
  q.kw = p.S - q.col0;
  q.kz = q.col0 == 0 ? 0 : q.kw;
  // in its band of the first step the row is on the grid while its column is below W (steps below kw and
  // below W - col0), in the next band from step kw on while the new column, k - kw, is below W
  const int w_left = p.W - q.col0;
  const uint32_t m0 = steps_below(q.kw < w_left ? q.kw : w_left);
  const uint32_t m1 = steps_below(q.kw + p.W) & ~steps_below(q.kw);
  q.in_grid = ((unsigned)q.bnd0 < (unsigned)rbands ? m0 : 0u) | ((unsigned)(q.bnd0 + 1) < (unsigned)rbands ? m1 : 0u);
  return q;
}
// The row by which a lane trails the head of the stream (block_pos): its own lane row -- except in a band of
// stacked images that holds several of them, where a row trails by its place in its own image: the images do not
// depend on each other, so the pipeline is only as deep as one image (two images of 7 rows: 7 steps instead of 14
// to fill and to drain, 35 instead of 42 steps for a stream of 8 such images).
__device__ __forceinline__ int skew_row(const ScanParams& p, int r) { return (p.stacked && r < p.rb) ? r % p.Himg : r; }   // (stacked: from 0, lane 0 is a row)
__device__ __forceinline__ int clamp_band(const ScanParams& p, int bnd) { return bnd < 0 ? 0 : (bnd >= p.nbands ? p.nbands - 1 : bnd); }
// Stages the operands of a block of kCK steps.  A is the position of the stream index (first step
// of the block) - 15; q and cell0 describe the lane's own row in that block (block_pos, and the cell
// index of its position at the first step: what the lane's copies fetch is what the lane itself will
// work on).  A wave copies the operands of one step of the block, wave % kCK (the waves that share a
// step take its copies in turn), so a lane works out one cell per block.
template <typename T, int NT, int CW, bool WITH_BOT, bool STAGE_X, int NWAVES, bool SKIP_BC = false>
__device__ __forceinline__ void stage_block(const ScanParams& p, char* buf, int b, Pos A, const BlockPos& q, int cell0,
                                            int e_wg0, int wave, int lane,
                                            const T* x0, const T* x1, const T* x2, const T* x3) {
  using SG = Stage<T, NT, CW, WITH_BOT>;
  constexpr bool BWD = WITH_BOT;
  static_assert(NWAVES % kCK == 0, "every step of a block needs a wave");
  constexpr int WPK = NWAVES / kCK;                       // waves per step
  const int ks = wave & (kCK - 1), wsub = wave / kCK;     // (uniform) the wave's step, its turn among the waves of that step
  // Source addresses are computed for every chunk and replaced by the page of zeros where the
  // chunk is not a cell of the grid (selects, no divergent branches).  Cells of one image are
  // addressed by 32-bit byte offsets from the image's base.
  const int64_t img = (int64_t)b * p.Hs * p.W;
  const char* zeros = reinterpret_cast<const char*>(p.zeros);
  const char* bc_img = reinterpret_cast<const char*>(p.bt + img * p.bc_stride);
  const int cstep = p.flip ? -1 : 1;                      // cells per column
  const int wrapc = (p.rb * p.W - p.S) * cstep;            // extra cells of a position reached through a band change
  const int slot = lane >> kHBShift;
  auto cell_at = [&](int k) { return cell0 + k * cstep + (k >= q.kw ? wrapc : 0); };
  auto ok_at = [&](int k) { return ((q.in_grid >> k) & 1u) != 0; };
  const int cell = cell_at(ks);
  const bool ok = ok_at(ks);
  char* kbuf = buf + ks * SG::kKStr;
  // The constants of the 16 lane rows at this step: gate offsets (log2 of the coefficient that is
  // folded into the gate) and input coefficients, with the cases of the grid's first row, of column 0
  // and of the ghost lanes worked out here, once per row and step, instead of in every lane that
  // sweeps the row.  Lanes read them back as one float4 (offT, offL, cT, cL).
  if (wsub == 0) {
    const int r = lane & (kHB - 1);
    const LaneK K = lane_consts<BWD>(p, clamp_band(p, ks >= q.kw ? q.bnd0 + 1 : q.bnd0), r, true);
    const bool col0 = q.kz == ks;
    const float4 kk = make_float4(col0 ? K.oT0 : K.oT, col0 ? -__builtin_huge_valf() : K.oL, col0 ? K.cT0 : K.cT, col0 ? K.cL0 : K.cL);
    if (slot == 0) *reinterpret_cast<float4*>(kbuf + SG::kConstPlane * SG::kPlane + r * 16) = kk;
  }
  // B_T, B_L, C: a copy moves the four state groups (lane >> 4) of one tensor for the 16 lane rows
  if constexpr (!SKIP_BC) {
#pragma unroll
    for (int tsr = 0; tsr < 3; ++tsr)
      if (tsr % WPK == wsub) {
        const uint32_t off = (uint32_t)cell * (uint32_t)(p.bc_stride * 4) + (uint32_t)(tsr * kN * 4 + slot * 16);
        lds_fill16<false>(ok ? bc_img + off : zeros, kbuf + tsr * 4 * SG::kPlane);
      }
  }
  if constexpr (STAGE_X) {
    const int64_t img_bytes = img * p.E * (int64_t)sizeof(T);
    if constexpr (SG::kCpt >= 4) {   // one step per copy: lanes = (channel chunk, row)
      constexpr int per = SG::kCpt / 4;                    // copies per tensor and step
#pragma unroll
      for (int tau = 0; tau < NT; ++tau) {
        const T* base = tau == 0 ? x0 : (tau == 1 ? x1 : (tau == 2 ? x2 : x3));
        const char* t_img = reinterpret_cast<const char*>(base) + img_bytes;
#pragma unroll
        for (int i = 0; i < per; ++i)
          if ((3 + tau * per + i) % WPK == wsub) {
            const int ch = e_wg0 + (i * 4 + slot) * SG::kElem;
            const uint32_t off = (uint32_t)(cell * p.E + ch) * (uint32_t)sizeof(T);
            lds_fill16<false>((ok && ch < p.E) ? t_img + off : zeros,
                              buf + SG::kXOff + tau * SG::kXTauBytes + ks * SG::kXStepBytes + i * 1024);
          }
      }
    } else if constexpr (SG::kCpt == 1) {   // all four steps per copy: lanes = (step, row); tensor tau is copied by the wave of step tau
      static_assert(kCK == 4 && NT <= kCK, "a wave-wide copy is the four steps of one tensor");
      const int cell4 = cell_at(slot);
      const int e_chunk = e_wg0 & ~(SG::kElem - 1);   // (a workgroup of fewer channels than a chunk copies the chunk they are in)
      const bool ok4 = ok_at(slot) && e_chunk < p.E;
      const uint32_t off = (uint32_t)(cell4 * p.E + e_chunk) * (uint32_t)sizeof(T);
#pragma unroll
      for (int tau = 0; tau < NT; ++tau)
        if (ks == tau && wsub == 0) {
          const T* base = tau == 0 ? x0 : (tau == 1 ? x1 : (tau == 2 ? x2 : x3));
          const char* t_img = reinterpret_cast<const char*>(base) + img_bytes;
          lds_fill16<false>(ok4 ? t_img + off : zeros, buf + SG::kXOff + tau * SG::kXTauBytes);
        }
    } else {                         // two steps per copy: lanes = (step, channel chunk, row); the wave of the even step copies
      static_assert(SG::kCpt == 2, "two chunks of channels per cell");
      if ((ks & 1) == 0) {
        const bool hi = lane >= 32;
        const int cell2 = hi ? cell_at(ks + 1) : cell;
        const bool ok2 = hi ? ok_at(ks + 1) : ok;
        const int ch = e_wg0 + (slot & 1) * SG::kElem;
        const uint32_t off = (uint32_t)(cell2 * p.E + ch) * (uint32_t)sizeof(T);
#pragma unroll
        for (int tau = 0; tau < NT; ++tau) {
          const T* base = tau == 0 ? x0 : (tau == 1 ? x1 : (tau == 2 ? x2 : x3));
          const char* t_img = reinterpret_cast<const char*>(base) + img_bytes;
          lds_fill16<false>((ok2 && ch < p.E) ? t_img + off : zeros, buf + SG::kXOff + tau * SG::kXTauBytes + ks * SG::kXStepBytes);
        }
      }
    }
  }
  // boundary rows were written earlier in this launch (or by the forward launch): read them
  // past the L1.  One wave-wide copy moves the four state groups (lane >> 4) of 16 channels at one step.
#pragma unroll
  for (int g = 0; g < SG::kG16; ++g)
    if ((3 + g) % WPK == wsub) {
      const int ch = e_wg0 + g * 16 + (lane & (kHB - 1));
      const Pos qa = pos_after(p, A, ks + (kHB - 1));    // the upper ghost is lane 0
      const float* src = p.zeros;
      if (!p.stacked && qa.bnd >= 1 && qa.bnd < p.nbands && qa.col < p.W && ch < p.E)
        src = p.top + ((((int64_t)(qa.bnd - 1) * p.B + b) * p.W + qa.col) * p.E + ch) * kN + slot * 4;
      lds_fill16<true>(src, kbuf + (SG::kTopPlane + 4 * g) * SG::kPlane);
    }
  if constexpr (WITH_BOT) {
#pragma unroll
    for (int g = 0; g < SG::kG16; ++g)
      if ((3 + SG::kG16 + g) % WPK == wsub) {
        const int ch = e_wg0 + g * 16 + (lane & (kHB - 1));
        const Pos qa = pos_after(p, A, ks);              // the lower ghost is lane 15
        const float* src = p.zeros;
        if (!p.stacked && qa.bnd >= 0 && qa.bnd + 1 < p.nbands && qa.col < p.W && ch < p.E)
          src = p.bot + (qa.bnd + 1) * p.bot_stride + (((int64_t)b * p.W + qa.col) * p.E + ch) * kN + slot * 4;
        lds_fill16<true>(src, kbuf + (SG::kBotPlane + 4 * g) * SG::kPlane);
      }
  }
}

// B_T, B_L, C straight from the caller's tensors, with no packed fp32 copy made first.
// 16-bit tensors (both passes): copied as they are into a small buffer of their own two blocks ahead
// (bc_raw_copy: one wave-wide copy moves the 16 rows of two (step, tensor) pairs, 32 bytes a row),
// and widened from there into the planes of the next block's staging buffer, in fold order (spos),
// while the current block is worked on (bc_widen): LDS to LDS, so that no wait for a vector load
// ever stands between a block's stores.
// fp32 tensors (forward without snapshots only): copied into the planes like every other operand,
// one block ahead (bc_direct_copy); the records keep the natural order of the states, which the
// forward kernel allows for in the order of its copy of A.
constexpr int kRawBytes = kCK * 3 * kHB * kN * 2;   // 16-bit B_T, B_L, C of one block: 6 KB
template <typename T, int CW, int NWAVES>
__device__ __forceinline__ void bc_direct_copy(const ScanParams& p, const void* const* tensors, char* buf, int b, const BlockPos& q,
                                               int cell0, int wave, int lane) {
  using SG = Stage<T, 3, CW, false>;
  static_assert(sizeof(T) == 4, "fp32 records need no widening");
  constexpr int WPK = NWAVES / kCK;
  const int ks = wave & (kCK - 1), wsub = wave / kCK;
  const int cstep = p.flip ? -1 : 1;
  const int cell = cell0 + ks * cstep + (ks >= q.kw ? (p.rb * p.W - p.S) * cstep : 0);
  const bool ok = ((q.in_grid >> ks) & 1u) != 0;
  const int slot = lane >> kHBShift;
  const int64_t img_bytes = (int64_t)b * p.Hs * p.W * (kN * (int64_t)sizeof(T));
#pragma unroll
  for (int tsr = 0; tsr < 3; ++tsr)
    if (tsr % WPK == wsub) {
      const char* t_img = static_cast<const char*>(tensors[tsr]) + img_bytes;
      lds_fill16<false>(ok ? t_img + ((uint32_t)cell * 64u + (uint32_t)slot * 16u) : reinterpret_cast<const char*>(p.zeros),
                        buf + ks * SG::kKStr + tsr * 4 * SG::kPlane);
    }
}
// q, cell0: the lane's row in the block to copy (block_pos); `live` false: zeros (there is no such block)
template <int NWAVES>
__device__ __forceinline__ void bc_raw_copy(const ScanParams& p, const void* const* tensors, char* raw, int b, const BlockPos& q,
                                            int cell0, int wave, int lane, bool live) {
  const int cstep = p.flip ? -1 : 1;
  const int wrapc = (p.rb * p.W - p.S) * cstep;
  const int sel = lane >> 5, hf = (lane >> kHBShift) & 1;
  const int64_t img_bytes = (int64_t)b * p.Hs * p.W * (kN * 2);
  for (int j = wave; j < kCK * 3 / 2; j += NWAVES) {   // (uniform) pairs (2j, 2j+1) of (step, tensor) = (c / 3, c % 3)
    const int c0 = 2 * j, c1 = 2 * j + 1;
    const int k = sel ? c1 / 3 : c0 / 3;
    const char* t0 = static_cast<const char*>(tensors[c0 % 3]);
    const char* t1 = static_cast<const char*>(tensors[c1 % 3]);
    const int cell = cell0 + k * cstep + (k >= q.kw ? wrapc : 0);
    const bool ok = live && ((q.in_grid >> k) & 1u) != 0;
    const char* src = (sel ? t1 : t0) + img_bytes + ((uint32_t)cell * 32u + (uint32_t)hf * 16u);
    lds_fill16<false>(ok ? src : reinterpret_cast<const char*>(p.zeros), raw + j * 1024);
  }
}
template <typename SG, int NWAVES>
__device__ __forceinline__ void bc_widen(const char* raw, char* buf, int wave, int lane) {
  const int r = lane & (kHB - 1), qd = lane >> kHBShift;   // row, four consecutive states 4*qd + m
  // state 4*qd + m belongs at position 4*m + perm(qd) of its record: word perm(qd) of plane m
  const int word = qd == 1 ? 2 : (qd == 2 ? 1 : qd);
  static_assert(spos<true>(4) == 2 && spos<true>(8) == 1 && spos<true>(13) == 7, "fold order");
  for (int c = wave; c < kCK * 3; c += NWAVES) {            // (uniform) (step, tensor) pairs
    const int k = c / 3, tsr = c - 3 * k;
    const uint2 v = *reinterpret_cast<const uint2*>(raw + c * 512 + (qd >> 1) * 256 + r * 16 + (qd & 1) * 8);
    float* dst = reinterpret_cast<float*>(buf + k * SG::kKStr + tsr * 4 * SG::kPlane + r * 16 + word * 4);
    dst[0 * SG::kPlane / 4] = __uint_as_float(v.x << 16);
    dst[1 * SG::kPlane / 4] = __uint_as_float(v.x & 0xffff0000u);
    dst[2 * SG::kPlane / 4] = __uint_as_float(v.y << 16);
    dst[3 * SG::kPlane / 4] = __uint_as_float(v.y & 0xffff0000u);
  }
}

// A workgroup of the linked sweep whose results mean nothing (Link::broken) says so in the caller's tensors: it
// overwrites its band's rows of up to three (B,H,W,E) tensors, for its own channels, with NaN, so that the failure
// shows without anyone reading the error word.
template <typename T>
__device__ __forceinline__ void poison_band(const ScanParams& p, int band, int b, int e_wg0, int cw, void* t0, void* t1, void* t2) {
  const int n = band_rows(p, band) * p.W * cw;
  const float nan = __builtin_nanf("");
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const int c = i % cw, at = i / cw;
    if (e_wg0 + c >= p.E) continue;
    const int cell = cell_of(p, band, at / p.W + 1, at % p.W);   // (lane row = row of the band + 1)
    const int64_t el = ((int64_t)b * p.Hs * p.W + cell) * p.E + e_wg0 + c;
    IO<T>::st(static_cast<T*>(t0) + el, nan);
    if (t1) IO<T>::st(static_cast<T*>(t1) + el, nan);
    if (t2) IO<T>::st(static_cast<T*>(t2) + el, nan);
  }
}

// ------------------------------------------------------------------------------------ forward
// y on its way out (m2d_fwd_kernel).  A lane's y of one step is 2 or 4 bytes at a cell of its own row: stored
// from the lane, a wave's y of one step goes to 16 different cache lines, 8 bytes each, and these stores cost
// the kernel 3 % (inference) to 9 % (with the snapshot stores of a training forward) of its time.  Instead the
// lanes drop y into LDS, a window of 4 steps at a time, and once per block every thread stores 8 or 16 bytes: the
// channels of one wave at one cell, so that the 8 (4) threads of a cell write its 64 (32) bytes together.
//   [wave][step of the window][lane row] chunks of the wave's channels (a wave's region is padded so that the
//   same chunk of consecutive waves sits in different banks).  Where the cells are in the image, the threads read
//   from a table that every lane fills once per block: byte offset of its row's cell at the block's first step,
//   the step at which the row changes band, the steps at which it is on the grid (all lanes of a row write the
//   same; the flush reads what slot 0 wrote).
template <typename T, int EC, int NW>
struct YTile {
  static constexpr int kChunk = 4 * EC * (int)sizeof(T);            // bytes of a wave's channels at one cell: 8 or 16
  static constexpr int kRegion = kCK * kHB * kChunk + kChunk;       // one wave's part of a window
  static constexpr int kBytes = (NW * kRegion + 15) / 16 * 16;      // one window
  static constexpr int kTableBytes = 4 * 64 * 8;                    // where the rows are: 4 blocks x 64 lanes x (offset, steps on the grid)
  static_assert(kChunk == 8 || kChunk == 16, "a thread flushes one 8- or 16-byte chunk");
  static_assert(kCK * kHB == 64 && kCK == 4, "a window is 64 cells: one per thread and wave-chunk");
};
// A snapshot quad: the four states of one state group of a lane, as the forward keeps them for the
// backward.  fp32 tensors keep them as they are.  16-bit tensors keep them rounded to bf16: the
// reference rounds every state of its hidden-state tensor to the tensors' type (wf_cuda.cu:40-69 writes
// hs in scalar_t), here only the one state in four steps that a block restarts from is; the forward's
// snapshot stores were a quarter of the traffic of the whole training step.
// Stored with the non-temporal hint: the data is read back once, by the backward pass, long after it
// has left the caches, and as an ordinary store it costs the forward kernel 0.02 ms at B=128, E=64, 56x56.
typedef float f4v __attribute__((ext_vector_type(4)));
typedef unsigned int u2v __attribute__((ext_vector_type(2)));
template <typename T> struct Snap;
template <> struct Snap<float> {
  typedef f4v quad;
  static __device__ __forceinline__ quad pack(float a, float b, float c, float d) { return f4v{a, b, c, d}; }
  static __device__ __forceinline__ void store(quad* dst, float a, float b, float c, float d) { __builtin_nontemporal_store(pack(a, b, c, d), dst); }
  static __device__ __forceinline__ float4 load(const quad* src) { return widen(*src); }
  static __device__ __forceinline__ quad zero() { return f4v{0.f, 0.f, 0.f, 0.f}; }
  static __device__ __forceinline__ float4 widen(quad v) { return make_float4(v.x, v.y, v.z, v.w); }
  // two neighbouring quads (a half of the states)
  static __device__ __forceinline__ void load2(const quad* src, quad (&dst)[2]) { dst[0] = src[0]; dst[1] = src[1]; }
  static __device__ __forceinline__ void store2(quad* dst, quad a, quad b) { __builtin_nontemporal_store(a, dst); __builtin_nontemporal_store(b, dst + 1); }
};
template <> struct Snap<bf16_t> {
  typedef u2v quad;
  static __device__ __forceinline__ quad pack(float a, float b, float c, float d) {
    // (a vector conversion is one v_cvt_pk_bf16_f32 per pair; two scalar casts and an OR are four instructions)
    typedef float f2v __attribute__((ext_vector_type(2)));
    typedef __bf16 b2v __attribute__((ext_vector_type(2)));
    return u2v{__builtin_bit_cast(uint32_t, __builtin_convertvector((f2v){a, b}, b2v)),
               __builtin_bit_cast(uint32_t, __builtin_convertvector((f2v){c, d}, b2v))};
  }
  static __device__ __forceinline__ void store(quad* dst, float a, float b, float c, float d) { __builtin_nontemporal_store(pack(a, b, c, d), dst); }
  static __device__ __forceinline__ float4 load(const quad* src) { return widen(*src); }
  static __device__ __forceinline__ quad zero() { return u2v{0u, 0u}; }
  static __device__ __forceinline__ float4 widen(quad v) {
    return make_float4(__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u), __uint_as_float(v.y << 16), __uint_as_float(v.y & 0xffff0000u));
  }
  // two neighbouring quads (a half of the states): one 16-byte piece
  typedef unsigned int u4v __attribute__((ext_vector_type(4)));
  static __device__ __forceinline__ void load2(const quad* src, quad (&dst)[2]) {
    const u4v v = *reinterpret_cast<const u4v*>(src);
    dst[0] = u2v{v.x, v.y}; dst[1] = u2v{v.z, v.w};
  }
  static __device__ __forceinline__ void store2(quad* dst, quad a, quad b) { __builtin_nontemporal_store(u4v{a.x, a.y, b.x, b.y}, reinterpret_cast<u4v*>(dst)); }
};
// Inside the 64 quads of one channel's snapshot, the quads of lane row r: quad q (state group q) sits at
// snap_lane(r) + snap_quad(q).  The two quads of a half of the states (0, 1 and 2, 3) are neighbours, so that a lane
// moves them as one piece (16 bytes of bf16 states in one instruction): [half of the states][16 lane rows][2 quads].
__device__ __forceinline__ constexpr int snap_quad(int q) { return (q >> 1) * (2 * kHB) + (q & 1); }
__device__ __forceinline__ int snap_lane(int r) { return 2 * r; }
// first quad of the kept snapshot number mi (snapshot_index) of channel e of image b: [b][kept block][E][2 halves of the states][16 lane rows][2 quads]
// (nkept: kept snapshots per image, p.ck_nblk.  A kernel that only runs at the default interval passes p.nblk and
// the block itself: it then needs none of the interval's parameters, which would cost it scalar registers.)
template <typename T>
__device__ __forceinline__ typename Snap<T>::quad* snapshot_at(const ScanParams& p, int b, int mi, int e, int nkept) {
  return reinterpret_cast<typename Snap<T>::quad*>(p.ckpt) + (((int64_t)b * nkept + mi) * p.E + e) * (kN / 4 * kHB);
}
// Block m of a window that starts at block m_lo (the window of band `band` in the linked sweep, else the whole
// stream): is its snapshot kept, and which of the image's kept snapshots is it.
__device__ __forceinline__ bool snapshot_kept(const ScanParams& p, int m, int m_lo) { return ((m - m_lo) & ((1 << p.ck_shift) - 1)) == 0; }
template <bool SLICED>
__device__ __forceinline__ int snapshot_index(const ScanParams& p, int m, int m_lo, int band) {
  return SLICED ? band * p.ck_pb + ((m - m_lo) >> p.ck_shift) : (m >> p.ck_shift);
}
// Lanes are never masked in the forward: a grid row that is between bands, or a lane that is no
// grid row, works on zero operands (its records come from the page of zeros), which keeps its
// state finite and never reaches a cell of the grid: at column 0 the left gate is closed, and
// what the lane below hands to a cell comes from the cell above it.  Only stores are predicated.
// NW waves per workgroup: 8, or 4 where the batch is too small to give every compute unit a
// workgroup of 8 (each wave then has a SIMD to itself).
// HALF: a snapshot every 2 steps instead of every 4 (m2d_bwd2_kernel restarts from them), and one more behind the sweep.
// Workgroups of 4 waves (few workgroups: each wave has a SIMD to itself) get 4 more waves that only stage: positions,
// copies, the wait for the neighbouring band of a linked sweep, the flush of y, the cross-wave channel sums of the
// backward; the first 4 only sweep.  A lone wave gets through a step as fast as its chain of instructions allows, and a
// quarter of that chain was staging (B=64, E=64, 56x56 bf16 with the copies left out: forward 0.220 -> 0.166 ms, backward
// 0.550 -> 0.458 ms).  Both kinds run the same loop, compiled once per role, with the same barriers.
constexpr int kAll = 0, kSweeper = 1, kStager = 2;   // what a wave does: both, only sweep, only stage
constexpr int kWholeHelpers = 4;
template <int MODE, int NW, int EC = 1>
constexpr int whole_helpers() { return (MODE != kModeStacked && NW == kFwdHalfWaves && EC == 1) ? kWholeHelpers : 0; }
// ST: the type the snapshots are kept in (T; float for bf16 tensors where the caller asks for fp32 snapshots).
template <typename T, int EC, bool CKPT, bool WRITE_Y, bool STAGE_X, int MODE, int NW = kFwdWaves, bool HALF = false, typename ST = T>
__global__ __launch_bounds__((NW + whole_helpers<MODE, NW, EC>()) * 64) void m2d_fwd_kernel(const ScanParams pin) {
  constexpr bool SLICED = MODE == kModeSliced, STACKED = MODE == kModeStacked;
  static_assert(!HALF || (CKPT && !SLICED), "snapshots every 2 steps: kept by a forward of one stream per image or stack");
  ScanParams p = pin;   // (stacked images: the height is shortened below for a last, shorter stack)
  if constexpr (!STACKED) {   // lets the compiler drop what only stacked images need
    __builtin_assume(p.stacked == 0);
    __builtin_assume(p.rb == kRB);
    __builtin_assume(p.S >= kHB + kCK - 1);
  }
  constexpr int CS = 64 >> kHBShift;
  constexpr int CW = NW * CS * EC;
  constexpr bool PERM = true;
  constexpr bool AHEAD = EC == 1 && STAGE_X;   // operands of step t+1 are fetched from LDS during step t
  constexpr int NH = whole_helpers<MODE, NW, EC>();   // waves that only stage (then the first NW waves only sweep)
  constexpr int NSTG = NH ? NH : NW;                  // waves that share the copies of a block
  using SG = Stage<T, 3, CW, false>;
  extern __shared__ float4 smem[];
  char* lds = reinterpret_cast<char*>(smem);       // two staging buffers
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  int lb = SLICED ? (int)blockIdx.x : logical_block(p.nwg);   // (linked bands keep the launch order: a band waits for a lower index)
  int m_lo = 0, m_hi = p.nblk;                     // blocks of steps this workgroup sweeps
  int my_band = 0;
  LinkT<NH ? NW * 64 : 0> link;
  if constexpr (SLICED) {   // the window of one band
    const int per = p.B * p.bpb;
    my_band = lb / per;
    lb -= my_band * per;
    m_lo = my_band * p.sl_nbb;
    m_hi = m_lo + p.sl_nbb;
    link.mine = p.prog + ((int64_t)my_band * per + lb) * kLinkStride;
    link.dep = my_band > 0 ? link.mine - per * kLinkStride : nullptr;
    link.err = p.link_err;
    link.rig(p, my_band);
  }
  const int b = lb / p.bpb;
  const int e_wg0 = (lb % p.bpb) * CW;
  if constexpr (STACKED) {   // the last stack of the batch may hold fewer images
    const int nimg = p.Breal - b * p.ips < p.ips ? p.Breal - b * p.ips : p.ips;
    p.H = nimg * p.Himg;
    p.nbands = (p.H + p.rb - 1) / p.rb;
    p.rows_last = p.H - (p.nbands - 1) * p.rb;
  }
  const bool helper = NH && wave >= NW;            // (uniform) stages, never sweeps
  const bool stages = !NH || helper;
  const int swave = NH ? wave - NW : wave;         // the wave's turn among those that stage
  const int stid = NH ? (int)threadIdx.x - NW * 64 : (int)threadIdx.x;   // ... and the thread's among their threads
  const int slot = lane >> kHBShift, r = lane & (kHB - 1);
  const int rbands = row_bands(p, r);
  const int rk = STACKED ? skew_row(p, r) : r;     // the row by which the lane trails the head of the stream
  const int ch_loc = ((helper ? swave : wave) * CS + slot) * EC;   // first channel of the lane inside the workgroup
  const int e_raw = e_wg0 + ch_loc;
  const bool ch_ok = !helper && e_raw < p.E;       // idle lanes still take part in staging and barriers
  const int e0 = e_raw < p.E ? e_raw : p.E - EC;
  // every byte a lane may read is finite from the start (pads are never written again)
  for (int i = threadIdx.x; i < 2 * SG::kBytes / 16; i += (NW + NH) * 64) smem[i] = make_float4(0.f, 0.f, 0.f, 0.f);

  float a2t[EC][kN], a2l[EC][kN], dsk[EC];
#pragma unroll
  for (int c = 0; c < EC; ++c) {
    ld16f(p.A2T + (e0 + c) * kN, a2t[c]);
    ld16f(p.A2L + (e0 + c) * kN, a2l[c]);
    dsk[c] = p.Df[e0 + c];
  }
  // fp32 records in natural state order (B_T, B_L, C straight from the caller's tensors): position j
  // of a record holds state j, so the register that meets position j takes A of state j.
  constexpr bool WIDEN = sizeof(T) == 2;            // 16-bit records pass through a buffer of their own, in every forward
  const bool direct = (WIDEN || !CKPT) && p.bc_direct != 0;   // (uniform)
  if (!WIDEN && direct) {   // (never taken by a 16-bit kernel)
#pragma unroll
    for (int c = 0; c < EC; ++c) {
      float t[kN], l[kN];
#pragma unroll
      for (int n = 0; n < kN; ++n) { t[n] = a2t[c][n]; l[n] = a2l[c][n]; }
#pragma unroll
      for (int j = 0; j < kN; ++j) { a2t[c][sinv<PERM>(j)] = t[j]; a2l[c][sinv<PERM>(j)] = l[j]; }
    }
  }
  char* raw = lds + 2 * SG::kBytes;                 // [2][kRawBytes]
  // y leaves through LDS (see YTile) where a wave's channels at a cell are whole 8- or 16-byte chunks: the same
  // condition as for staging x
  constexpr bool YTILE = WRITE_Y && STAGE_X;
  using YT = YTile<T, EC, NW>;
  char* ywin = raw + (WIDEN ? 2 * kRawBytes : 0);   // [2 windows][YT::kBytes]
  uint2* ytab = reinterpret_cast<uint2*>(ywin + 2 * YT::kBytes);   // [block & 3][lane]
  if constexpr (YTILE) {   // the block before the first has no row on the grid
    for (int i = threadIdx.x; i < 4 * 64; i += (NW + NH) * 64) ytab[i] = make_uint2(0u, 0u);
  }

  settle_loads();
  __syncthreads();
  const T* X = static_cast<const T*>(p.x);
  const T* DT = static_cast<const T*>(p.dT);
  const T* DL = static_cast<const T*>(p.dL);
  const T* DY = DL;   // not staged by the forward (NT = 3)
  const float ninf = -__builtin_huge_valf();
  const int64_t img_cell0 = (int64_t)b * p.Hs * p.W;
  // (B,H,W,E) tensors are addressed as image base (uniform) + 32-bit byte offset (per lane)
  const int64_t img_bytes = img_cell0 * p.E * (int64_t)sizeof(T);
  char* Yimg = static_cast<char*>(p.y) + img_bytes;
  const char* Ximg = reinterpret_cast<const char*>(X) + img_bytes;
  const char* DTimg = reinterpret_cast<const char*>(DT) + img_bytes;
  const char* DLimg = reinterpret_cast<const char*>(DL) + img_bytes;
  const uint32_t estep = (uint32_t)(p.flip ? -p.E : p.E) * (uint32_t)sizeof(T);   // one column further

  const float g1 = !STACKED && r == 0 ? 1.f : 0.f;   // the ghost's T input coefficient
  const uint32_t wrap_adj = (uint32_t)(p.rb * p.W - p.S) * estep;   // extra offset of a cell reached through a band change

  // byte offsets of the lane's operand groups inside a staging buffer (step 0, group 0): a grid row
  // reads B_T, B_L, C of its cell; the ghost reads the row above as its B_T (and row 0 of the B_L and C
  // planes, zeros, as stand-ins for the other two, which it multiplies by 0)
  const uint32_t row_off = r * 16;
  const bool ghost = !STACKED && r == 0;   // (stacked images: no row above a band to replay, lane 0 is a row like the others)
  const uint32_t rec_off = ghost ? SG::top_off(ch_loc) : row_off;
  const uint32_t rec_cstep = ghost ? 16 : 0;   // the ghost reads a record per channel, grid rows share theirs
  const uint32_t xd_off = SG::kXOff + SG::x_off(r, ch_loc);
  constexpr uint32_t kXK = SG::kXStepBytes;   // XD bytes per step

  // per block: where the lane is and what depends on it
  BlockPos bp;
  uint32_t cell_off0 = 0;       // byte offset in a (H,W,E) image of the lane's cell at the first step of the block

  // Operands of one step, read from the staging buffer one step ahead of their use so that the
  // LDS latency hides behind the arithmetic of the step before.
  struct Ops {
    float xv[EC], dtv[EC], dlv[EC];
    float4 bt[EC][4], bl[4], cc[4];
    float4 kk;   // the row's constants at this step: gate offsets T, L and input coefficients T, L
  };
  auto fetch = [&](const char* bufc, int k, Ops& o) {
    if constexpr (STAGE_X) {
      const T* xr = reinterpret_cast<const T*>(bufc + xd_off + k * kXK);
      IO<T>::template ldv<EC>(xr, o.xv);
      IO<T>::template ldv<EC>(xr + SG::kXTauBytes / sizeof(T), o.dtv);
      IO<T>::template ldv<EC>(xr + 2 * SG::kXTauBytes / sizeof(T), o.dlv);
    } else {   // straight from memory, for the lane's position at step k of the current block
#pragma unroll
      for (int c = 0; c < EC; ++c) { o.xv[c] = 0.f; o.dtv[c] = 0.f; o.dlv[c] = 0.f; }
      if (ch_ok && ((bp.in_grid >> k) & 1u)) {
        const uint32_t off = cell_off0 + (uint32_t)k * estep + (k >= bp.kw ? wrap_adj : 0u);
        IO<T>::template ldv<EC>(reinterpret_cast<const T*>(Ximg + off), o.xv);
        IO<T>::template ldv<EC>(reinterpret_cast<const T*>(DTimg + off), o.dtv);
        IO<T>::template ldv<EC>(reinterpret_cast<const T*>(DLimg + off), o.dlv);
      }
    }
    const char* rec = bufc + rec_off + k * SG::kKStr;
    const char* row = bufc + row_off + k * SG::kKStr;
    o.kk = *reinterpret_cast<const float4*>(row + SG::kConstPlane * SG::kPlane);
#pragma unroll
    for (int c = 0; c < EC; ++c)
#pragma unroll
      for (int q = 0; q < 4; ++q) o.bt[c][q] = *reinterpret_cast<const float4*>(rec + c * rec_cstep + q * SG::kPlane);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      o.bl[q] = *reinterpret_cast<const float4*>(row + SG::kBLOff + q * SG::kPlane);
      o.cc[q] = WRITE_Y ? *reinterpret_cast<const float4*>(row + SG::kCOff + q * SG::kPlane) : make_float4(0, 0, 0, 0);
    }
  };

  float h[EC][kN];
#pragma unroll
  for (int c = 0; c < EC; ++c)
#pragma unroll
    for (int n = 0; n < kN; ++n) h[c][n] = 0.f;
  typename Snap<ST>::quad* ckp = nullptr;      // where the lane stores its snapshot in the first step of the current block
  typename Snap<ST>::quad* ckp2 = nullptr;     // ... and (HALF) in its third step
  int ypar = 0;                 // window that the current block fills
  const uint32_t y_lane_off = (uint32_t)(wave * YT::kRegion + (r * CS + slot) * EC * (int)sizeof(T));
  auto step = [&](int k, const Ops& o) {
    const float offT = o.kk.x, offL = o.kk.y, cT = o.kk.z, cL = o.kk.w;
    const bool inr = ch_ok && ((bp.in_grid >> k) & 1u);
    float yv[EC];
#pragma unroll
    for (int c = 0; c < EC; ++c) {
      const float sT = __builtin_fmaf(cT * o.dtv[c], o.xv[c], g1);
      const float sL = cL * o.dlv[c] * o.xv[c];
      float acc = 0.f;
      typename Snap<ST>::quad pend = Snap<ST>::zero();   // a quad that waits for its neighbour (16-bit snapshots: two bf16 quads leave as one 16-byte store)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float4 b4 = o.bt[c][q], l4 = o.bl[q], c4 = o.cc[q];
        const float bq[4] = {b4.x, b4.y, b4.z, b4.w}, lq[4] = {l4.x, l4.y, l4.z, l4.w}, cq[4] = {c4.x, c4.y, c4.z, c4.w};
        // The T gates first, then the L gates, then the four state chains: the multiply-add that
        // takes the state of the row above through DPP is inline assembly, which the compiler's
        // hazard recogniser does not see, and it must not issue right behind the v_exp that
        // produces its gate (a transcendental result needs one wait state before a VALU reads it).
        float aT[4], aL[4];
#pragma unroll
        for (int w = 0; w < 4; ++w) aT[w] = fexp2(__builtin_fmaf(o.dtv[c], a2t[c][sinv<PERM>(4 * q + w)], offT));
        pin4(aT);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int w = 0; w < 4; ++w) aL[w] = fexp2(__builtin_fmaf(o.dlv[c], a2l[c][sinv<PERM>(4 * q + w)], offL));
        pin4(aL);
        __builtin_amdgcn_sched_barrier(0);
        if (CKPT && (k == 0 || (HALF && k == 2))) {   // the four states as they are before this step: stored with their neighbours' quad
          const typename Snap<ST>::quad pk = Snap<ST>::pack(h[c][sinv<PERM>(4 * q)], h[c][sinv<PERM>(4 * q + 1)], h[c][sinv<PERM>(4 * q + 2)], h[c][sinv<PERM>(4 * q + 3)]);
          if ((q & 1) == 0) pend = pk;
          else Snap<ST>::store2((k == 0 ? ckp : ckp2) + c * (kN / 4 * kHB) + snap_quad(q - 1), pend, pk);
        }
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          const int n = sinv<PERM>(4 * q + w);
          float u = sL * lq[w];
          u = __builtin_fmaf(sT, bq[w], u);
          u = fma_row_below(aT[w], h[c][n], u);       // + aT * h of the row above (the lane below)
          const float hn = __builtin_fmaf(aL[w], h[c][n], u);
          h[c][n] = hn;
          if (WRITE_Y) acc = __builtin_fmaf(hn, cq[w], acc);
        }
      }
      yv[c] = __builtin_fmaf(o.xv[c], dsk[c], acc);
    }
    if (p.nbands > 1 && !p.stacked) {   // last row of a band: the next band's ghost will replay it
      const bool wk = k >= bp.kw;
      const int bk = wk ? bp.bnd0 + 1 : bp.bnd0;
      if (inr && r == kRB && bk + 1 < p.nbands) {
        const int ck = wk ? bp.col0 + k - p.S : bp.col0 + k;
        float4* tw = reinterpret_cast<float4*>(p.top + ((((int64_t)bk * p.B + b) * p.W + ck) * p.E + e0) * kN);
#pragma unroll
        for (int c = 0; c < EC; ++c)
#pragma unroll
          for (int q = 0; q < 4; ++q)
          {
            const float4 row = make_float4(h[c][sinv<PERM>(4 * q)], h[c][sinv<PERM>(4 * q + 1)], h[c][sinv<PERM>(4 * q + 2)], h[c][sinv<PERM>(4 * q + 3)]);
            if constexpr (SLICED) store_row_device_scope(tw + c * 4 + q, row); else tw[c * 4 + q] = row;
          }
      }
    }
    if constexpr (YTILE) {   // no branch: a lane off the grid drops its y too, next to an offset that says so
      // A window is flushed behind the barrier of its block.  With operands fetched a step ahead that barrier
      // stands before the block's last step, which therefore opens the next window.
      const int ks = AHEAD ? (k + 1) & (kCK - 1) : k;   // place of this step in its window
      char* win = ywin + (AHEAD && k == kCK - 1 ? ypar ^ 1 : ypar) * YT::kBytes;
      IO<T>::template stv<EC>(reinterpret_cast<T*>(win + y_lane_off + ks * (kHB * YT::kChunk)), yv);
    } else {
      if (WRITE_Y && inr)
        IO<T>::template stv<EC>(reinterpret_cast<T*>(Yimg + (cell_off0 + (uint32_t)k * estep + (k >= bp.kw ? wrap_adj : 0u))), yv);
    }
  };
  // One window of y from LDS to memory, after a barrier behind which every wave has written it: thread (cell c,
  // wave j) takes the channels of wave j at cell c.  first_only: just the first step of the window (the last
  // step of the sweep; the rest of the window is from two blocks ago).
  auto flush_y = [&](int par, int m, bool first_only) {   // m: the block whose barrier this is
    const char* win = ywin + par * YT::kBytes;
    const int c = stid / NW, j = stid % NW;
    const int ks = c >> kHBShift;                                  // the cell's step in the window ...
    const int k = AHEAD ? (ks + kCK - 1) & (kCK - 1) : ks;         // ... and in its block,
    const int blk = AHEAD && ks == 0 ? m - 1 : m;                  // which is the one before for the window's first step
    const uint2 row = ytab[(blk & 3) * 64 + (c & (kHB - 1))];
    const uint32_t off = row.x + (uint32_t)k * estep + (k >= (int)(row.y >> 8) ? wrap_adj : 0u);
    if (((row.y >> k) & 1u) && e_wg0 + j * CS * EC < p.E && !(first_only && c >= kHB)) {
      if constexpr (YT::kChunk == 8)
        *reinterpret_cast<uint2*>(Yimg + off + j * YT::kChunk) = *reinterpret_cast<const uint2*>(win + j * YT::kRegion + c * YT::kChunk);
      else
        *reinterpret_cast<uint4*>(Yimg + off + j * YT::kChunk) = *reinterpret_cast<const uint4*>(win + j * YT::kRegion + c * YT::kChunk);
    }
  };

  Pos A = pos_of(p, m_lo * kCK - (kHB - 1));     // position of the stream index t0 - 15 (wave-uniform)
  bp = block_pos(p, A, rk, rbands);
  int cell0 = cell_of(p, bp.bnd0, r, bp.col0);   // cell index of the lane's position at the first step of the block
  if constexpr (SLICED) { if (stages) link.wait_for(link_need_fwd(0, p.sl_nbb)); }
  BlockPos bpq = bp;     // 16-bit direct records: the block after the next (fetched two blocks ahead)
  int cellq = cell0;
  int rp = 0;            // ... and the half of `raw` it goes to
  if (direct) {
    if constexpr (WIDEN) {
      if (stages) bc_raw_copy<NSTG>(p, pin.bcd, raw, b, bp, cell0, swave, lane, true);
      bpq = block_pos(p, pos_after(p, A, kCK), rk, rbands);
      cellq = cell_of(p, bpq.bnd0, r, bpq.col0);
      if (stages) bc_raw_copy<NSTG>(p, pin.bcd, raw + kRawBytes, b, bpq, cellq, swave, lane, m_lo + 1 < m_hi);
    } else {
      if (stages) bc_direct_copy<T, CW, NSTG>(p, pin.bcd, lds, b, bp, cell0, swave, lane);
    }
    if (stages) stage_block<T, 3, CW, false, STAGE_X, NSTG, true>(p, lds, b, A, bp, cell0, e_wg0, swave, lane, X, DT, DL, DY);
    if constexpr (WIDEN) {
      staging_fence();
      if (stages) bc_widen<SG, NSTG>(raw, lds, swave, lane);
    }
  } else {
    if (stages) stage_block<T, 3, CW, false, STAGE_X, NSTG>(p, lds, b, A, bp, cell0, e_wg0, swave, lane, X, DT, DL, DY);
  }
  staging_fence();
  Ops opsA, opsB;
  if constexpr (AHEAD) { if (!helper) fetch(lds, 0, opsA); }
  int cur = 0;
  // The sweep over the blocks of the window, as a wave of the given role runs it.
  auto sweep = [&](auto role) {
  constexpr int ROLE = decltype(role)::value;
  constexpr bool STAGES = ROLE != kSweeper, SWEEPS = ROLE != kStager;
  for (int m = m_lo; m < m_hi; ++m) {
    const bool last = m + 1 == m_hi;
    // the next block: where the lane's row will be is also what the lane's copies fetch
    const Pos An = pos_after(p, A, kCK);
    BlockPos bpn;
    int celln;
    if (WIDEN && direct && EC == 1) {   // the next block was worked out a block ago; its records are in `raw` already
      bpn = bpq;
      celln = cellq;
      bpq = block_pos(p, pos_after(p, An, kCK), rk, rbands);
      cellq = cell_of(p, bpq.bnd0, r, bpq.col0);
      if constexpr (STAGES) bc_raw_copy<NSTG>(p, pin.bcd, raw + rp * kRawBytes, b, bpq, cellq, swave, lane, m + 2 < m_hi);
    } else if (WIDEN && direct) {   // two channels per lane: no registers to carry a block's positions in; worked out twice
      bpn = block_pos(p, An, rk, rbands);
      celln = cell_of(p, bpn.bnd0, r, bpn.col0);
      if constexpr (STAGES) {
        const BlockPos q2 = block_pos(p, pos_after(p, An, kCK), rk, rbands);
        bc_raw_copy<NSTG>(p, pin.bcd, raw + rp * kRawBytes, b, q2, cell_of(p, q2.bnd0, r, q2.col0), swave, lane, m + 2 < m_hi);
      }
    } else {
      bpn = block_pos(p, An, rk, rbands);
      celln = cell_of(p, bpn.bnd0, r, bpn.col0);
    }
    if (STAGES && !last) {
      if constexpr (SLICED) link.wait_for(link_need_fwd(m + 1 - m_lo, p.sl_nbb));
      if (direct) {
        if constexpr (!WIDEN) bc_direct_copy<T, CW, NSTG>(p, pin.bcd, lds + (cur ^ 1) * SG::kBytes, b, bpn, celln, swave, lane);
        stage_block<T, 3, CW, false, STAGE_X, NSTG, true>(p, lds + (cur ^ 1) * SG::kBytes, b, An, bpn, celln, e_wg0, swave, lane, X, DT, DL, DY);
        if constexpr (WIDEN) bc_widen<SG, NSTG>(raw + (rp ^ 1) * kRawBytes, lds + (cur ^ 1) * SG::kBytes, swave, lane);
      } else {
        stage_block<T, 3, CW, false, STAGE_X, NSTG>(p, lds + (cur ^ 1) * SG::kBytes, b, An, bpn, celln, e_wg0, swave, lane, X, DT, DL, DY);
      }
    }
    rp ^= 1;
    if constexpr (!SWEEPS) {   // a wave that only stages: its copies have landed, then what follows the block's barrier
      staging_landed();
      __syncthreads();
      if constexpr (SLICED) link.publish((uint32_t)(m - m_lo + 1));
      if constexpr (YTILE) flush_y(ypar, m, false);
    } else {
    cell_off0 = (uint32_t)(cell0 * p.E + e0) * (uint32_t)sizeof(T);
    if constexpr (YTILE)
      ytab[(m & 3) * 64 + lane] = make_uint2((uint32_t)(cell0 * p.E + e_wg0) * (uint32_t)sizeof(T), ((uint32_t)(bp.kw < kCK ? bp.kw : kCK) << 8) | (bp.in_grid & 15u));
    // Snapshot of the state before the block (after step t0-1).  The stores are issued inside the
    // first step, each group of four states just before it is overwritten: the waves of the whole
    // grid run in step, and one burst of all snapshots would stall them.  Every lane stores, with no
    // branch inside the step (a predicate per lane splits the step into five scheduling regions:
    // 0.292 against 0.281 ms at B=128, E=64, 56x56).  Only the lanes whose previous position was a
    // cell of the grid hold something the backward needs (snapshot_lane), and only those it reads;
    // the other lanes write to their own place all the same.  Channels past E, whose place is
    // another channel's, and blocks whose snapshot is not kept (block 0; a longer checkpoint
    // interval) write to the image's place for block 0, which nobody reads.
    if constexpr (CKPT && HALF) {   // snapshots 2m and 2m + 1 (snapshot 0, the state before the sweep, is the place nobody reads)
      ckp = snapshot_at<ST>(p, b, (m > 0 && ch_ok) ? 2 * m : 0, e0, p.ck_nblk) + snap_lane(r);
      ckp2 = snapshot_at<ST>(p, b, ch_ok ? 2 * m + 1 : 0, e0, p.ck_nblk) + snap_lane(r);
    } else if constexpr (CKPT) {
      const bool keep = m > 0 && snapshot_kept(p, m, m_lo);
      ckp = snapshot_at<ST>(p, b, (keep && ch_ok) ? snapshot_index<SLICED>(p, m, m_lo, my_band) : 0, e0, p.ck_nblk) + snap_lane(r);
    }
    const char* bufc = lds + cur * SG::kBytes;
    const char* bufn = lds + (cur ^ 1) * SG::kBytes;
    // (uniform) some lane writes y at each of the first three steps: the wave issues at least
    // three stores between the copies for the next block and the barrier that ends this one
    // (y that leaves through LDS is stored once per block, before the copies for the next block: nothing to count)
    const bool y_thrice = WRITE_Y && !YTILE && __any(ch_ok && (bp.in_grid & 7u) == 7u);
    // (uniform, linked sweep) lane 14 stores the band's last row at each of the first three steps
    const bool top_thrice = SLICED && __any(ch_ok && (bp.in_grid & 7u) == 7u && r == kRB && bp.kw >= kCK && bp.bnd0 + 1 < p.nbands);
    auto next_block_landed = [&] {
      // the stores issued since (snapshot, y) need not have completed, only the copies before them
      // (a wave that only sweeps has issued no copies, but waits all the same: with it, every store older than a block
      // has completed, which the boundary rows that a later band of this workgroup reads back rely on)
      if constexpr (SLICED) {
        // Linked sweep: the band below needs, of the newest block it is told about, the last row of the steps 0 and 1
        // only (link_need_fwd).  Only what is issued after the row of step 1 stays in flight (y of step 1, row and
        // y of step 2), so that this block counts as done at its end.
        if (top_thrice) {
          if (y_thrice) staging_landed_behind<4 * EC + 2>(); else staging_landed_behind<4 * EC>();
        } else {
          if (y_thrice) staging_landed_behind<2>(); else staging_landed();
        }
      } else if constexpr (CKPT) {
        // snapshot stores of the steps before the last: per channel and snapshot two 16-byte pieces of bf16 quads or four fp32 quads
        // (counting too few only waits longer, too many reads operands that have not landed; the wait's field counts to 15)
        constexpr int kSnaps = (HALF ? 2 : 1) * EC * (sizeof(ST) == 2 ? 2 : 4);
        if (y_thrice) staging_landed_behind<(kSnaps + 3 < 15 ? kSnaps + 3 : 15)>(); else staging_landed_behind<(kSnaps < 15 ? kSnaps : 15)>();
      } else {
        if (y_thrice) staging_landed_behind<3>(); else staging_landed();
      }
    };
    if constexpr (AHEAD) {
      static_assert(kCK % 2 == 0, "the two operand sets alternate and must close over a block");
#pragma unroll
      for (int k = 0; k < kCK; ++k) {
        Ops& now = (k & 1) ? opsB : opsA;
        Ops& ahead = (k & 1) ? opsA : opsB;
        if (k + 1 < kCK) {
          fetch(bufc, k + 1, ahead);
        } else {
          // Last step of the block: its operands are in registers already, so the buffer can be
          // handed over now.  The copies of the next block have landed in every wave after this
          // barrier, and no wave reads the current buffer any more.
          next_block_landed();
          __syncthreads();
          lead_if_younger<NW>(wave, true);   // (from here to the second step of the next block: half of the way to the next barrier)
          // every wave has waited for the rows it stored at the steps 0 and 1 of this block
          if constexpr (SLICED && STAGES) link.publish((uint32_t)(m - m_lo + 1));
          if constexpr (YTILE && STAGES) flush_y(ypar, m, false);   // the last step of the block before and the first three of this one
          if (!last) fetch(bufn, 0, ahead);
        }
        if (k == 1) lead_if_younger<NW>(wave, false);
        step(k, now);   // also past the end of the sweep (last block): zero operands like any position off the grid, nothing stored
      }
    } else {
#pragma unroll
      for (int k = 0; k < kCK; ++k) {
        // The operands of the next block must have landed before the barrier that ends this
        // block.  Waiting here, before the stores of the last step are issued, keeps the latency
        // of those stores off the critical path (the counter covers loads and stores alike).
        if (k == kCK - 1) next_block_landed();
        if (k == 0 || k == kCK / 2) lead_if_younger<NW>(wave, k == 0);
        fetch(bufc, k, opsA);
        step(k, opsA);
      }
      __syncthreads();
      if constexpr (SLICED && STAGES) link.publish((uint32_t)(m - m_lo + 1));
      if constexpr (YTILE && STAGES) flush_y(ypar, m, false);   // the four steps of this block
    }
    }
    ypar ^= 1;
    cur ^= 1;
    A = An;
    bp = bpn;
    cell0 = celln;
  }
  };
  if constexpr (NH == 0) sweep(std::integral_constant<int, kAll>{});
  else if (helper) sweep(std::integral_constant<int, kStager>{});
  else sweep(std::integral_constant<int, kSweeper>{});
  if constexpr (YTILE && AHEAD) {   // the last step of the sweep
    __syncthreads();
    if (stages) flush_y(ypar, m_hi, true);
  }
  if constexpr (CKPT && HALF) if (!helper) {   // the state behind the last block: what the last step of the sweep left is among it
    typename Snap<ST>::quad* end = snapshot_at<ST>(p, b, ch_ok ? 2 * p.nblk : 0, e0, p.ck_nblk) + snap_lane(r);
#pragma unroll
    for (int c = 0; c < EC; ++c)
#pragma unroll
      for (int q = 0; q < 4; q += 2)
        Snap<ST>::store2(end + c * (kN / 4 * kHB) + snap_quad(q),
                        Snap<ST>::pack(h[c][sinv<PERM>(4 * q)], h[c][sinv<PERM>(4 * q + 1)], h[c][sinv<PERM>(4 * q + 2)], h[c][sinv<PERM>(4 * q + 3)]),
                        Snap<ST>::pack(h[c][sinv<PERM>(4 * q + 4)], h[c][sinv<PERM>(4 * q + 5)], h[c][sinv<PERM>(4 * q + 6)], h[c][sinv<PERM>(4 * q + 7)]));
  }
  if constexpr (SLICED) {   // the whole window is done once every store of every wave has completed
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    link.publish((uint32_t)p.sl_nbb);
    bool broken = link.broken();
    if constexpr (NH > 0) {   // only the waves that wait know: they tell the others (the staging buffers are free now)
      if ((int)threadIdx.x == link.pub) *reinterpret_cast<volatile uint32_t*>(lds) = broken ? 1u : 0u;
      __syncthreads();
      broken = *reinterpret_cast<volatile uint32_t*>(lds) != 0u;
    }
    if (WRITE_Y && broken) poison_band<T>(p, my_band, b, e_wg0, CW, p.y, nullptr, nullptr);
  }
}

// ------------------------------------------------------- forward, the states of a channel split over lanes
// Few images leave most of the device idle with the kernel above (a wave per 4 channels of an
// image), and a sweep then takes as long as one wave needs for its chain of instructions.  Here the
// 16 states of ONE channel are split over the 4 lane groups of a wave (lane = (state group g, row r),
// 4 states per lane): four times as many waves, each with about a third of the instructions per
// step.  A workgroup has 8 waves = 8 channels.  Staging, schedules and memory formats are those of
// m2d_fwd_kernel; y of a cell is the sum over the 4 lane groups (two lane-swap steps), stored by group 0.
constexpr int kSplitWaves = 8;
constexpr int kSplitHalfWaves = 4;   // where workgroups of 8 would leave compute units idle
// Workgroups of 4 waves: a step of a wave that has a SIMD to itself takes as long as its chain of
// instructions, and of those under a third are the step's arithmetic; the rest stages the next block (positions,
// addresses, copies, the wait for the neighbouring band).  So such a workgroup gets 4 more waves that do nothing but
// stage (and, in the backward, add up the channel sums of every step), one to a SIMD beside a wave that does nothing
// but sweep: the two chains run side by side.
// Workgroups of 8 sweeping waves have the same 4 (3 waves to a SIMD, 168 registers a lane: 1024x1024x64 fp32 forward
// 2.29 -> 2.10 ms, backward 4.97 -> 4.39; 32 images of 56x56x64 bf16, one stream each, 0.146 -> 0.134 and 0.338 ->
// 0.284), except where rows are not whole 16-byte chunks (SX false: the compiler's
// register allocator fails on those kernels at 768 threads).  With 8 more the backward no longer fits the registers
// of a lane at 4 waves to a SIMD and ran a quarter slower.
constexpr int kSplitHelpers = 4;
template <int MODE, int NWS, bool SX = true>
constexpr int split_helpers() { return (NWS == kSplitHalfWaves || SX) ? kSplitHelpers : 0; }
__device__ __forceinline__ float sum_over_groups(float v) {
  v = fold16(v, v);
  return fold32(v, v);
}
template <typename T, bool CKPT, bool WRITE_Y, bool STAGE_X, int MODE, int NWS = kSplitWaves>
__global__ __launch_bounds__((NWS + split_helpers<MODE, NWS, STAGE_X>()) * 64) void m2d_fwd_split_kernel(const ScanParams pin) {
  static_assert(MODE != kModeStacked, "stacked images are many: they never need the split");
  constexpr bool SLICED = MODE == kModeSliced;
  const ScanParams& p = pin;
  __builtin_assume(p.stacked == 0);
  __builtin_assume(p.rb == kRB);
  __builtin_assume(p.S >= kHB + kCK - 1);
  constexpr int NW = NWS, CW = NW;
  constexpr int NH = split_helpers<MODE, NWS, STAGE_X>();   // waves that only stage (then the first NW waves only sweep)
  constexpr int NSTG = NH ? NH : NW;               // waves that share the copies of a block
  using SG = Stage<T, 3, CW, false>;
  constexpr bool WIDEN = sizeof(T) == 2;
  extern __shared__ float4 smem[];
  char* lds = reinterpret_cast<char*>(smem);       // two staging buffers
  char* raw = lds + 2 * SG::kBytes;                // [2][kRawBytes] (16-bit B_T, B_L, C on their way)
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  int lb = SLICED ? (int)blockIdx.x : logical_block(p.nwg);
  int m_lo = 0, m_hi = p.nblk;
  int my_band = 0;
  LinkT<NH ? NW * 64 : 0> link;
  if constexpr (SLICED) {
    const int per = p.B * p.bpb;
    my_band = lb / per;
    lb -= my_band * per;
    m_lo = my_band * p.sl_nbb;
    m_hi = m_lo + p.sl_nbb;
    link.mine = p.prog + ((int64_t)my_band * per + lb) * kLinkStride;
    link.dep = my_band > 0 ? link.mine - per * kLinkStride : nullptr;
    link.err = p.link_err;
    link.rig(p, my_band);
  }
  const bool helper = NH && wave >= NW;             // (uniform) stages, never sweeps
  const bool stages = !NH || helper;
  const int swave = NH ? wave - NW : wave;          // the wave's turn among those that stage
  const int b = lb / p.bpb;
  const int e_wg0 = (lb % p.bpb) * CW;
  const int g = lane >> kHBShift, r = lane & (kHB - 1);   // state group, lane row
  const int rbands = row_bands(p, r);
  const int ch_loc = helper ? 0 : wave;             // the wave's channel inside the workgroup
  const bool ch_ok = !helper && e_wg0 + ch_loc < p.E;   // (uniform) idle waves still take part in staging and barriers
  const int e0 = ch_ok ? e_wg0 + ch_loc : p.E - 1;
  for (int i = threadIdx.x; i < 2 * SG::kBytes / 16; i += (NW + NH) * 64) smem[i] = make_float4(0.f, 0.f, 0.f, 0.f);

  // Position 4g + w of a record is met by register w: state sinv(4g + w) in fold order, state 4g + w
  // where the records come straight from fp32 tensors (natural order).
  const bool direct = (WIDEN || !CKPT) && p.bc_direct != 0;   // (uniform)
  float a2t[4], a2l[4];
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const int q = w == 1 ? 2 : (w == 2 ? 1 : w);   // sinv<true>(4g + w) = q * 4 + g
    const int n = (!WIDEN && direct) ? 4 * g + w : q * 4 + g;
    a2t[w] = p.A2T[e0 * kN + n];
    a2l[w] = p.A2L[e0 * kN + n];
  }
  static_assert(sinv<true>(1) == 8 && sinv<true>(6) == 5 && sinv<true>(15) == 15, "fold order");
  const float dsk = p.Df[e0];
  settle_loads();
  __syncthreads();

  const T* X = static_cast<const T*>(p.x);
  const T* DT = static_cast<const T*>(p.dT);
  const T* DL = static_cast<const T*>(p.dL);
  const T* DY = DL;
  const int64_t img_cell0 = (int64_t)b * p.Hs * p.W;
  const int64_t img_bytes = img_cell0 * p.E * (int64_t)sizeof(T);
  char* Yimg = static_cast<char*>(p.y) + img_bytes;
  const char* Ximg = reinterpret_cast<const char*>(X) + img_bytes;
  const char* DTimg = reinterpret_cast<const char*>(DT) + img_bytes;
  const char* DLimg = reinterpret_cast<const char*>(DL) + img_bytes;
  const uint32_t estep = (uint32_t)(p.flip ? -p.E : p.E) * (uint32_t)sizeof(T);
  const uint32_t wrap_adj = (uint32_t)(p.rb * p.W - p.S) * estep;
  const float g1 = r == 0 ? 1.f : 0.f;             // the ghost's T input coefficient

  // the lane's group of B_T (the ghost: of the row above), of B_L and C (the ghost: zeros of its own row)
  const uint32_t row_off = r * 16 + g * SG::kPlane;
  const uint32_t rec_off = r == 0 ? SG::top_off(ch_loc) + g * SG::kPlane : row_off;
  const uint32_t const_off = SG::kConstPlane * SG::kPlane + r * 16;
  const uint32_t xd_off = SG::kXOff + SG::x_off(r, ch_loc + (CW < SG::kElem ? e_wg0 & (SG::kElem - 1) : 0));   // (4 channels of a 16-bit tensor: their half of the chunk)
  constexpr uint32_t kXK = SG::kXStepBytes;

  BlockPos bp;
  uint32_t cell_off0 = 0;
  float h[4] = {0.f, 0.f, 0.f, 0.f};
  typename Snap<T>::quad* ckp = nullptr;

  auto step = [&](const char* bufc, int k) {
    float xv = 0.f, dtv = 0.f, dlv = 0.f;
    const bool inr = ch_ok && ((bp.in_grid >> k) & 1u);
    const uint32_t goff = cell_off0 + (uint32_t)k * estep + (k >= bp.kw ? wrap_adj : 0u);
    if constexpr (STAGE_X) {
      const T* xr = reinterpret_cast<const T*>(bufc + xd_off + k * kXK);
      xv = IO<T>::ld(xr); dtv = IO<T>::ld(xr + SG::kXTauBytes / sizeof(T)); dlv = IO<T>::ld(xr + 2 * SG::kXTauBytes / sizeof(T));
    } else if (inr) {
      xv = IO<T>::ld(reinterpret_cast<const T*>(Ximg + goff));
      dtv = IO<T>::ld(reinterpret_cast<const T*>(DTimg + goff));
      dlv = IO<T>::ld(reinterpret_cast<const T*>(DLimg + goff));
    }
    const float4 kk = *reinterpret_cast<const float4*>(bufc + const_off + k * SG::kKStr);
    const float4 b4 = *reinterpret_cast<const float4*>(bufc + rec_off + k * SG::kKStr);
    const float4 l4 = *reinterpret_cast<const float4*>(bufc + row_off + SG::kBLOff + k * SG::kKStr);
    const float4 c4 = WRITE_Y ? *reinterpret_cast<const float4*>(bufc + row_off + SG::kCOff + k * SG::kKStr) : make_float4(0, 0, 0, 0);
    const float offT = kk.x, offL = kk.y, cT = kk.z, cL = kk.w;
    const float bq[4] = {b4.x, b4.y, b4.z, b4.w}, lq[4] = {l4.x, l4.y, l4.z, l4.w}, cq[4] = {c4.x, c4.y, c4.z, c4.w};
    const float sT = __builtin_fmaf(cT * dtv, xv, g1);
    const float sL = cL * dlv * xv;
    // gates before chains (see m2d_fwd_kernel: no DPP multiply-add right behind the v_exp that makes its gate)
    float aT[4], aL[4];
#pragma unroll
    for (int w = 0; w < 4; ++w) aT[w] = fexp2(__builtin_fmaf(dtv, a2t[w], offT));
    pin4(aT);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int w = 0; w < 4; ++w) aL[w] = fexp2(__builtin_fmaf(dlv, a2l[w], offL));
    pin4(aL);
    __builtin_amdgcn_sched_barrier(0);
    if (CKPT && k == 0) Snap<T>::store(ckp, h[0], h[1], h[2], h[3]);   // the lane's states as they are before this step
    float acc = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      float u = sL * lq[w];
      u = __builtin_fmaf(sT, bq[w], u);
      u = fma_row_below(aT[w], h[w], u);
      const float hn = __builtin_fmaf(aL[w], h[w], u);
      h[w] = hn;
      if (WRITE_Y) acc = __builtin_fmaf(hn, cq[w], acc);
    }
    if (p.nbands > 1) {   // last row of a band: the next band's ghost will replay it
      const bool wk = k >= bp.kw;
      const int bk = wk ? bp.bnd0 + 1 : bp.bnd0;
      if (inr && r == kRB && bk + 1 < p.nbands) {
        const int ck = wk ? bp.col0 + k - p.S : bp.col0 + k;
        float4* tw = reinterpret_cast<float4*>(p.top + ((((int64_t)bk * p.B + b) * p.W + ck) * p.E + e0) * kN) + g;
        const float4 row = make_float4(h[0], h[1], h[2], h[3]);
        if constexpr (SLICED) store_row_device_scope(tw, row); else *tw = row;
      }
    }
    if constexpr (WRITE_Y) {
      const float yv = __builtin_fmaf(xv, dsk, sum_over_groups(acc));
      if (inr && g == 0) IO<T>::st(reinterpret_cast<T*>(Yimg + goff), yv);
    }
  };

  Pos A = pos_of(p, m_lo * kCK - (kHB - 1));     // position of the stream index t0 - 15 (wave-uniform)
  bp = block_pos(p, A, r, rbands);
  int cell0 = cell_of(p, bp.bnd0, r, bp.col0);
  if constexpr (SLICED) { if (stages) link.wait_for(link_need_fwd(0, p.sl_nbb)); }
  BlockPos bpq = bp;     // 16-bit direct records: the block after the next (fetched two blocks ahead)
  int cellq = cell0;
  int rp = 0;
  if (direct) {
    if constexpr (WIDEN) {
      if (stages) bc_raw_copy<NSTG>(p, pin.bcd, raw, b, bp, cell0, swave, lane, true);
      bpq = block_pos(p, pos_after(p, A, kCK), r, rbands);
      cellq = cell_of(p, bpq.bnd0, r, bpq.col0);
      if (stages) bc_raw_copy<NSTG>(p, pin.bcd, raw + kRawBytes, b, bpq, cellq, swave, lane, m_lo + 1 < m_hi);
    } else {
      if (stages) bc_direct_copy<T, CW, NSTG>(p, pin.bcd, lds, b, bp, cell0, swave, lane);
    }
    if (stages) stage_block<T, 3, CW, false, STAGE_X, NSTG, true>(p, lds, b, A, bp, cell0, e_wg0, swave, lane, X, DT, DL, DY);
    if constexpr (WIDEN) {
      staging_fence();
      if (stages) bc_widen<SG, NSTG>(raw, lds, swave, lane);
    }
  } else {
    if (stages) stage_block<T, 3, CW, false, STAGE_X, NSTG>(p, lds, b, A, bp, cell0, e_wg0, swave, lane, X, DT, DL, DY);
  }
  staging_fence();
  int cur = 0;
  // The sweep over the blocks of the window, as a wave of the given role runs it: kAll stages and sweeps; with waves
  // that only stage, those run it as kStager and the others as kSweeper, each with its own part of the work and all
  // with the same barriers.
  auto sweep = [&](auto role) {
  constexpr int ROLE = decltype(role)::value;
  constexpr bool STAGES = ROLE != kSweeper, SWEEPS = ROLE != kStager;
  for (int m = m_lo; m < m_hi; ++m) {
    const bool last = m + 1 == m_hi;
    const Pos An = pos_after(p, A, kCK);
    BlockPos bpn;
    int celln;
    if (WIDEN && direct) {
      bpn = bpq;
      celln = cellq;
      bpq = block_pos(p, pos_after(p, An, kCK), r, rbands);
      cellq = cell_of(p, bpq.bnd0, r, bpq.col0);
      if constexpr (STAGES) bc_raw_copy<NSTG>(p, pin.bcd, raw + rp * kRawBytes, b, bpq, cellq, swave, lane, m + 2 < m_hi);
    } else {
      bpn = block_pos(p, An, r, rbands);
      celln = cell_of(p, bpn.bnd0, r, bpn.col0);
    }
    if (STAGES && !last) {
      if constexpr (SLICED) link.wait_for(link_need_fwd(m + 1 - m_lo, p.sl_nbb));
      if (direct) {
        if constexpr (!WIDEN) bc_direct_copy<T, CW, NSTG>(p, pin.bcd, lds + (cur ^ 1) * SG::kBytes, b, bpn, celln, swave, lane);
        stage_block<T, 3, CW, false, STAGE_X, NSTG, true>(p, lds + (cur ^ 1) * SG::kBytes, b, An, bpn, celln, e_wg0, swave, lane, X, DT, DL, DY);
        if constexpr (WIDEN) bc_widen<SG, NSTG>(raw + (rp ^ 1) * kRawBytes, lds + (cur ^ 1) * SG::kBytes, swave, lane);
      } else {
        stage_block<T, 3, CW, false, STAGE_X, NSTG>(p, lds + (cur ^ 1) * SG::kBytes, b, An, bpn, celln, e_wg0, swave, lane, X, DT, DL, DY);
      }
    }
    rp ^= 1;
    if constexpr (SWEEPS) {
    cell_off0 = (uint32_t)(cell0 * p.E + e0) * (uint32_t)sizeof(T);
    if constexpr (CKPT) {   // every lane stores, without a branch inside the step: see m2d_fwd_kernel
      const bool keep = m > 0 && snapshot_kept(p, m, m_lo);
      ckp = snapshot_at<T>(p, b, (keep && ch_ok) ? snapshot_index<SLICED>(p, m, m_lo, my_band) : 0, e0, p.ck_nblk) + snap_lane(r) + snap_quad(g);
    }
    const char* bufc = lds + cur * SG::kBytes;
    // (uniform) stores that the wave is sure to issue in the first three steps, after the copies for the
    // next block: y where some lane is on the grid at all three, the boundary row where the band's last row
    // is and another band follows.  They need not have completed when the block ends, only the copies.
    const bool on3 = ch_ok && (bp.in_grid & 7u) == 7u;
    const bool y_thrice = WRITE_Y && __any(on3);
    const bool top_thrice = p.nbands > 1 && __any(on3 && r == kRB && bp.kw >= kCK && bp.bnd0 + 1 < p.nbands);
    // Linked sweep: the band below needs, of the newest block it is told about, the boundary rows of the steps 0 and
    // 1 only (link_need_fwd).  With just the stores issued after those of step 1 left in flight (y of step 1, row and
    // y of step 2), this block counts as done at its end.
    const int younger = SLICED ? (y_thrice ? 2 : 0) + (top_thrice ? 1 : 0)
                               : (CKPT ? 1 : 0) + (y_thrice ? 3 : 0) + (top_thrice ? 3 : 0);
#pragma unroll
    for (int k = 0; k < kCK; ++k) {
      if (k == kCK - 1) staging_landed_behind_n(younger);
      if (k == 0 || k == kCK / 2) lead_if_younger<NW>(wave, k == 0);
      step(bufc, k);
    }
    } else {
      staging_landed();   // the next block's operands are in place
    }
    __syncthreads();
    if constexpr (SLICED && STAGES) link.publish((uint32_t)(m - m_lo + 1));
    cur ^= 1;
    A = An;
    bp = bpn;
    cell0 = celln;
  }
  };
  if constexpr (NH == 0) sweep(std::integral_constant<int, kAll>{});
  else if (helper) sweep(std::integral_constant<int, kStager>{});
  else sweep(std::integral_constant<int, kSweeper>{});
  if constexpr (SLICED) {
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    link.publish((uint32_t)p.sl_nbb);
    bool broken = link.broken();
    if constexpr (NH > 0) {   // only the waves that wait know: they tell the others (the staging buffers are free now)
      if ((int)threadIdx.x == link.pub) *reinterpret_cast<volatile uint32_t*>(lds) = broken ? 1u : 0u;
      __syncthreads();
      broken = *reinterpret_cast<volatile uint32_t*>(lds) != 0u;
    }
    if (WRITE_Y && broken) poison_band<T>(p, my_band, b, e_wg0, CW, p.y, nullptr, nullptr);
  }
}

// ----------------------------------------------------------------------------------- backward
// Channel sums by lane-swap butterflies.  The wave holds 4 channel slots; for a group of 4 states
// every lane lists its values v[0..3] and fold16(fold32(v0,v1), fold32(v2,v3)) leaves, in the
// lane of slot 0,2,1,3, the sum over all slots of the value at position 0,1,2,3.
// fold_state(m, qi) is the state to list at position qi of group m so that afterwards slot q
// holds state q*4 + m.
__device__ __forceinline__ constexpr int fold_state(int m, int qi) {
  const int q = (qi == 1) ? 2 : (qi == 2) ? 1 : qi;
  return q * 4 + m;
}

// Exchange buffers of the backward kernel (channel sums across the waves of a workgroup), in units
// of one (step, half of the states) buffer of [wave][3][64] float2.  Where the LDS has room for one
// buffer per step of a block (kCK), the sums of a half are exchanged in one go after its kCK adjoint
// steps: two barriers per half instead of one per step.  Otherwise two buffers are used alternately
// with one barrier per step.
template <typename T, int NW>
constexpr int bwd_exchange_sets() {
  return sizeof(float2) * kCK * NW * 3 * 64 + sizeof(float) * NW * 4 * 2 * kN + 256 +
         2 * (size_t)Stage<T, 4, NW * 4, true>::kBytes + (sizeof(T) == 2 ? 2 * kRawBytes : 0) <= 160 * 1024 ? kCK : 2;
}
// As in the forward, lanes are never masked: rows outside the grid and cells outside the row work
// on zero operands.  For the adjoint this means that a row which has not reached its last column
// yet keeps lambda = mu = 0 exactly, and that a row past column 0 carries finite values that are
// multiplied by zero coefficients (delta, dy, x are zero there) wherever they meet a sum.
// NW waves per workgroup: 8, or 4 for small batches (see the forward kernel).  With 4 waves a thread
// of the first three adds up both components of one lane's pair of channel sums.
// REPLAY: the forward kept a snapshot for the first block only of every group of 2^ck_shift blocks (a longer
// checkpoint interval).  Before the sweep enters a group, at its last block, the forward is replayed over the
// group's other blocks from that snapshot, one block at a time through the idle staging buffer, and the state
// before each block is parked in the workgroup's ring in memory, where the sweep then finds it like a snapshot.
// A lane reads back only what it wrote itself.
template <typename T, bool STAGE_X, int MODE, int NW = kBwdWaves, bool REPLAY = false, typename ST = T>
__global__ __launch_bounds__((NW + (REPLAY ? 0 : whole_helpers<MODE, NW>())) * 64) void m2d_bwd_kernel(const ScanParams pin) {
  constexpr bool SLICED = MODE == kModeSliced, STACKED = MODE == kModeStacked;
  ScanParams p = pin;   // (stacked images: the height is shortened below for a last, shorter stack)
  if constexpr (!STACKED) {   // lets the compiler drop what only stacked images need
    __builtin_assume(p.stacked == 0);
    __builtin_assume(p.rb == kRB);
    __builtin_assume(p.S >= kHB + kCK - 1);
  }
  constexpr int CS = 64 >> kHBShift;     // 4 channel slots
  constexpr int SLOT = 3 * 64;           // float2s per wave in one exchange buffer
  constexpr int CW = NW * CS;
  constexpr bool PERM = true;
  constexpr int NH = REPLAY ? 0 : whole_helpers<MODE, NW>();   // waves that only stage and add up the channel sums (then the first NW waves only sweep)
  constexpr int NSTG = NH ? NH : NW;                           // waves that share the copies of a block and the sums of a half
  using SG = Stage<T, 4, CW, true>;
  extern __shared__ float4 smem[];
  // Exchange buffers for the channel sums of one (step, half of the states).  Either one per step of
  // a block (BATCH): the waves fill them during the kCK adjoint steps of a half, meet at a barrier,
  // add up, and meet again before the next half fills them.  Or two, used alternately, with one
  // barrier per step (a buffer is rewritten two exchanges later, after a barrier that every wave
  // reaches only once it has finished reading it).
  constexpr int XSETS = bwd_exchange_sets<T, NW>();
  constexpr bool BATCH = XSETS == kCK;
  static_assert(NH == 0 || BATCH, "the waves that stage add up the sums of a half in one go");
  float2* slots = reinterpret_cast<float2*>(smem);                       // [XSETS][wave][3][64]
  float* a_lds = reinterpret_cast<float*>(slots + XSETS * NW * SLOT);    // [wave][CS][2][16], fold order
  char* lds = reinterpret_cast<char*>(a_lds + NW * CS * 2 * kN);  // 2 staging buffers
  constexpr bool WIDEN = sizeof(T) == 2;    // 16-bit B_T, B_L, C can come straight from the caller's tensors (bc_raw_copy, bc_widen)
  char* raw = lds + 2 * SG::kBytes;         // [2][kRawBytes] for them
  const bool direct = WIDEN && p.bc_direct != 0;   // (uniform)
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  int lb = SLICED ? (int)blockIdx.x : logical_block(p.nwg);   // (linked bands keep the launch order: a band waits for a lower index)
  int m_lo = 0, m_hi = p.nblk;              // blocks of steps this workgroup sweeps (from m_hi - 1 down to m_lo)
  int my_band = 0;
  LinkT<NH ? NW * 64 : 0> link;
  if constexpr (SLICED) {   // the window of one band; the bands are launched from the last to the first
    const int per = p.B * p.bpb;
    const int kk = lb / per;
    lb -= kk * per;
    my_band = p.nbands - 1 - kk;
    m_lo = my_band * p.sl_nbb;
    m_hi = m_lo + p.sl_nbb;
    link.mine = p.prog + ((int64_t)my_band * per + lb) * kLinkStride;
    link.dep = my_band + 1 < p.nbands ? link.mine + per * kLinkStride : nullptr;
    link.err = p.link_err;
    link.rig(p, my_band);
  }
  const int b = lb / p.bpb;
  const int eg = lb % p.bpb;
  if constexpr (STACKED) {   // the last stack of the batch may hold fewer images
    const int nimg = p.Breal - b * p.ips < p.ips ? p.Breal - b * p.ips : p.ips;
    p.H = nimg * p.Himg;
    p.nbands = (p.H + p.rb - 1) / p.rb;
    p.rows_last = p.H - (p.nbands - 1) * p.rb;
  }
  const int e_wg0 = eg * CW;
  const bool helper = NH && wave >= NW;      // (uniform) stages and adds up, never sweeps
  const bool stages = !NH || helper;
  const int swave = NH ? wave - NW : wave;   // the wave's turn among those that stage
  const int slot = lane >> kHBShift, r = lane & (kHB - 1);
  const int rbands = row_bands(p, r);
  const int rk = STACKED ? skew_row(p, r) : r;     // the row by which the lane trails the head of the stream
  const int ch_loc = (helper ? swave : wave) * CS + slot;
  const int e_raw = e_wg0 + ch_loc;
  const bool ch_ok = !helper && e_raw < p.E;   // padding lanes/waves still take part in the barriers
  const int e = e_raw < p.E ? e_raw : p.E - 1;
  if (!helper) {  // A of the wave's channels into LDS in fold order (read back group by group)
    float* mine = a_lds + ch_loc * (2 * kN);
    mine[spos<true>(r)] = p.A2T[e * kN + r];
    mine[kN + spos<true>(r)] = p.A2L[e * kN + r];
  }
  // planes that no copy writes must hold finite values from the start
  for (int i = threadIdx.x; i < 2 * SG::kBytes / 16; i += (NW + NH) * 64) reinterpret_cast<float4*>(lds)[i] = make_float4(0.f, 0.f, 0.f, 0.f);
  const uint32_t a_base_off = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) float*)(a_lds + ch_loc * (2 * kN)));
  const float dsk = p.Df[e];
  settle_loads();

  const T* X = static_cast<const T*>(p.x);
  const T* DT = static_cast<const T*>(p.dT);
  const T* DL = static_cast<const T*>(p.dL);
  const T* DY = static_cast<const T*>(p.dy);
  const float ninf = -__builtin_huge_valf();
  const int64_t img_cell0 = (int64_t)b * p.Hs * p.W;
  // (B,H,W,E) tensors: image base (uniform) + 32-bit byte offset (per lane)
  const int64_t img_bytes = img_cell0 * p.E * (int64_t)sizeof(T);
  const char* Ximg = reinterpret_cast<const char*>(X) + img_bytes;
  const char* DTimg = reinterpret_cast<const char*>(DT) + img_bytes;
  const char* DLimg = reinterpret_cast<const char*>(DL) + img_bytes;
  const char* DYimg = reinterpret_cast<const char*>(DY) + img_bytes;
  char* DXimg = static_cast<char*>(p.dx) + img_bytes;
  char* DDTimg = static_cast<char*>(p.ddT) + img_bytes;
  char* DDLimg = static_cast<char*>(p.ddL) + img_bytes;
  char* BOTimg = reinterpret_cast<char*>(p.bot + (int64_t)b * p.W * p.E * kN);   // + band * bot_stride
  // per-workgroup channel sums: [channel group][cell][C, B_T, B_L][16]
  char* PARTimg = reinterpret_cast<char*>(p.part + ((int64_t)eg * p.Ptot + img_cell0) * (3 * kN));

  float accAT[kN], accAL[kN], accD = 0.f;
  float muT[kN], muL[kN];
#pragma unroll
  for (int n = 0; n < kN; ++n) { accAT[n] = 0.f; accAL[n] = 0.f; muT[n] = 0.f; muL[n] = 0.f; }
  // byte offsets of the lane's operand record inside a staging buffer at step 0 of a block, and
  // its advance per step: a grid row reads (B_T, B_L, C) of its cell; the upper ghost (lane 0)
  // reads the row above as its B_T; the lower ghost (lane 15) reads the row of mu_T below as its C.
  // The neighbouring records that a ghost reads in the other two places are finite and meet zeros.
  // The other two reads of a ghost land 4 and 8 planes from its boundary row: boundary rows of other
  // channels, operands of other rows or planes nobody writes, finite all of them, and they meet zeros.
  const uint32_t rec_off = STACKED ? r * 16 : (r == 0 ? SG::top_off(ch_loc) : (r == kHB - 1 ? SG::bot_off(ch_loc) - SG::kCOff : r * 16));
  const uint32_t xd_off = SG::kXOff + SG::x_off(r, ch_loc);
  constexpr uint32_t kXK = SG::kXStepBytes;   // XD bytes per step
  // The sum that this thread adds up in the exchange belongs to its own lane row r: one float of
  // the float2 of the lane (slot f_s, row r) for tensor f_v (a whole float2 where a workgroup has
  // fewer threads than sums).  The first 6 (3) waves do the adding.
  constexpr bool PAIRS = NW * 64 < 2 * SLOT;   // fewer threads than sums: a thread takes a pair
  const int f_combo = wave * 4 + slot;
  const bool f_on = f_combo < (PAIRS ? 12 : 24);
  const int f_v = PAIRS ? f_combo >> 2 : f_combo >> 3, f_s = PAIRS ? f_combo & 3 : (f_combo >> 1) & 3;
  const int f_comp = PAIRS ? 0 : f_combo & 1;
  const int f_it = f_v * 64 + f_s * kHB + r;
  const uint32_t f_sub = (uint32_t)(f_v * kN + f_s * 4 + f_comp) * (uint32_t)sizeof(float);
  const float g1 = !STACKED && r == 0 ? 1.f : 0.f;   // (stacked images: all 16 lanes are rows, see grid_row)

  const uint32_t estep = (uint32_t)(p.flip ? -p.E : p.E) * (uint32_t)sizeof(T);   // one column further
  const uint32_t wrap_adj = (uint32_t)(p.rb * p.W - p.S) * estep;   // extra offset of a cell reached through a band change
  const uint32_t pstep = (uint32_t)(p.flip ? -1 : 1) * (uint32_t)(3 * kN * sizeof(float));
  const uint32_t pwrap_adj = (uint32_t)(p.rb * p.W - p.S) * pstep;

  // per block: where the lane (and the lane row whose sums this thread adds up) is, and what
  // depends on it
  BlockPos bp;
  // 1 on the lower ghost: lambda = 1 * (row of mu_T below), which is staged as zeros where there is no band below
  const float gb1 = !STACKED && r == kHB - 1 ? 1.f : 0.f;
  const uint32_t row_const_off = SG::kConstPlane * SG::kPlane + r * 16;   // the row's constants at step 0 of a staging buffer
  uint32_t cell_off0 = 0;       // byte offset in a (H,W,E) image of the lane's cell at the first step of the block
  uint32_t f_off0 = 0;          // byte offset in the channel-sum image of this thread's sum at the first step
  // state snapshot at the start of the block whose position A is given (zero for lanes that were not under way)
  // (kept as it comes from memory until the block starts: nothing waits for the loads before then)
  typename Snap<ST>::quad cknext[4];
  // The replaying kernel of 8 waves (256 registers per lane) fetches the snapshot of a block when the block starts,
  // not during the block before: the registers that would hold it meanwhile are what the kernel lacks, and waiting
  // for the fetch costs less than spilling in the sweep (B=128, E=64, 56x56, interval 8: 1.05 against 1.10 ms).
  // Workgroups of 4 waves have the registers (512x512, interval 8: 4.47 against 4.66 ms).
  constexpr bool LATE_SNAPSHOT = REPLAY && NW == kBwdWaves;
  constexpr int kRingSlot = CW * (kN / 4) * kHB;   // quads of one parked snapshot of the workgroup
  // place of block mm in its group of 2^ck_shift blocks (0: the forward kept its snapshot)
  auto member = [&](int mm) { return REPLAY ? (mm - m_lo) & ((1 << p.ck_shift) - 1) : 0; };
  // Where the lane finds the state before block mm: a (uniform) base, in the checkpoints or in the workgroup's ring
  // [member - 1][channel of the workgroup][state group][row], plus the same offset of the lane in both (channels
  // past E point at the last channel's place: they park nothing and use nothing).
  auto snapshot_of_lane = [&](int mm) {
    if constexpr (!REPLAY) {   // the default interval: a snapshot for every block, as before
      return snapshot_at<ST>(p, b, mm, e, p.nblk) + snap_lane(r);
    } else {
      const int mem = member(mm);
      typename Snap<ST>::quad* base =
          mem != 0 ? static_cast<typename Snap<ST>::quad*>(p.ring) + ((int64_t)blockIdx.x * ((1 << p.ck_shift) - 1) + (mem - 1)) * kRingSlot - e_wg0 * (kN / 4 * kHB)
                   : snapshot_at<ST>(p, b, snapshot_index<SLICED>(p, mm, m_lo, my_band), 0, p.ck_nblk);
      return base + (e * (kN / 4 * kHB) + snap_lane(r));
    }
  };
  // the sweep enters a group at block mm, and the block has no snapshot: the replay brings its state
  auto opens_group = [&](int mm) { return REPLAY && member(mm) != 0 && (mm == m_hi - 1 || member(mm) == (1 << p.ck_shift) - 1); };
  auto load_ckpt = [&](int mm, bool take) {   // take: the forward kept the lane's state before block mm
    if (mm == 0 || !take) {
#pragma unroll
      for (int q = 0; q < 4; ++q) cknext[q] = Snap<ST>::zero();
    } else {
      const typename Snap<ST>::quad* ck = snapshot_of_lane(mm);
#pragma unroll
      for (int q = 0; q < 4; q += 2) Snap<ST>::load2(ck + snap_quad(q), *reinterpret_cast<typename Snap<ST>::quad(*)[2]>(&cknext[q]));
    }
  };
  auto pos_before = [&](Pos Q) {   // kCK positions earlier
    Q.col -= kCK;
    if (Q.col < 0) { Q.col += p.S; Q.bnd -= 1; }
    return Q;
  };

  Pos A = pos_of(p, (m_hi - 1) * kCK - (kHB - 1));   // position of the stream index t0 - 15 (wave-uniform)
  __syncthreads();   // the zeros are in place before the first copies land on them
  bp = block_pos(p, A, rk, rbands);
  int cell0 = cell_of(p, bp.bnd0, r, bp.col0);   // cell index of the lane's position at the first step of the block
  bool ck_take = snapshot_lane(p, Pos{bp.bnd0, bp.col0}, r, ch_ok);   // the lane restores a snapshot for the block to come
  if (!LATE_SNAPSHOT && !opens_group(m_hi - 1)) load_ckpt(m_hi - 1, ck_take);   // (else: after the replay that opens the first iteration)
  if constexpr (SLICED) { if (stages) link.wait_for(link_need_bwd(p.sl_nbb - 1, p.sl_nbb)); }
  // the lane's row in the block two before (A2 = position of that block): what its raw copies fetch
  auto raw_copy_for = [&](Pos A2, char* dst, bool live) {
    const BlockPos q2 = block_pos(p, A2, rk, rbands);
    bc_raw_copy<NSTG>(p, pin.bcd, dst, b, q2, cell_of(p, q2.bnd0, r, q2.col0), swave, lane, live);
  };
  int rp = 0;   // half of `raw` that the next raw copy goes to
  if (direct) {
    if (stages) bc_raw_copy<NSTG>(p, pin.bcd, raw, b, bp, cell0, swave, lane, true);
    if (stages) raw_copy_for(pos_before(A), raw + kRawBytes, m_hi - 2 >= m_lo);
    if (stages) stage_block<T, 4, CW, true, STAGE_X, NSTG, true>(p, lds, b, A, bp, cell0, e_wg0, swave, lane, X, DT, DL, DY);
    staging_fence();
    if (stages) bc_widen<SG, NSTG>(raw, lds, swave, lane);
  } else {
    if (stages) stage_block<T, 4, CW, true, STAGE_X, NSTG>(p, lds, b, A, bp, cell0, e_wg0, swave, lane, X, DT, DL, DY);
  }
  staging_fence();
  int cur = 0;
  int xpar = 0;   // exchange buffer in use

  // The sweep over the blocks of the window, as a wave of the given role runs it (see m2d_fwd_kernel).
  auto sweep = [&](auto role) {
  constexpr int ROLE = decltype(role)::value;
  constexpr bool STAGES = ROLE != kSweeper, SWEEPS = ROLE != kStager;
  for (int m = m_hi - 1; m >= m_lo; --m) {
    const int t0 = m * kCK;
    const char* bufc = lds + cur * SG::kBytes;
    if constexpr (REPLAY) {
      // The sweep enters a group of blocks at a block without a snapshot: replay the forward from the group's first
      // block up to this one.  The other staging buffer is idle (the operands of this block are in `bufc`, those of
      // the block before are fetched further down), and so is the half of `raw` that the next raw copy goes to.
      if (opens_group(m)) {
        const int mem = member(m);
        char* bufr = lds + (cur ^ 1) * SG::kBytes;
        float hq[kN];   // hq[4 * mg + qi]: state fold_state(mg, qi), the order of the snapshot quads
        for (int q = m - mem; q < m; ++q) {   // (uniform)
          const Pos Aq = pos_of(p, q * kCK - (kHB - 1));
          const BlockPos bq = block_pos(p, Aq, rk, rbands);
          const int cellq = cell_of(p, bq.bnd0, r, bq.col0);
          if (direct) {
            bc_raw_copy<NW>(p, pin.bcd, raw + rp * kRawBytes, b, bq, cellq, wave, lane, true);
            stage_block<T, 4, CW, true, STAGE_X, NW, true>(p, bufr, b, Aq, bq, cellq, e_wg0, wave, lane, X, DT, DL, DY);
            staging_fence();
            bc_widen<SG, NW>(raw + rp * kRawBytes, bufr, wave, lane);
          } else {
            stage_block<T, 4, CW, true, STAGE_X, NW>(p, bufr, b, Aq, bq, cellq, e_wg0, wave, lane, X, DT, DL, DY);
          }
          staging_fence();
          // the states before block q: the kept snapshot for the first block of the group, else what the replay of
          // the block before left, and zero in both cases for a lane that was not under way (see snapshot_lane)
          const bool take_q = q != 0 && snapshot_lane(p, Pos{bq.bnd0, bq.col0}, r, ch_ok);
          if (q == m - mem) {
            const typename Snap<ST>::quad* ck = snapshot_of_lane(q);
#pragma unroll
            for (int mg = 0; mg < 4; ++mg) {
              const float4 v = take_q ? Snap<ST>::load(ck + snap_quad(mg)) : make_float4(0.f, 0.f, 0.f, 0.f);
              hq[4 * mg + 0] = v.x; hq[4 * mg + 1] = v.y; hq[4 * mg + 2] = v.z; hq[4 * mg + 3] = v.w;
            }
          } else {
#pragma unroll
            for (int n = 0; n < kN; ++n) hq[n] = take_q ? hq[n] : 0.f;
          }
          const uint32_t cell_offq = (uint32_t)(cellq * p.E + e) * (uint32_t)sizeof(T);
#pragma unroll
          for (int k = 0; k < kCK; ++k) {
            const float4 kk = *reinterpret_cast<const float4*>(bufr + (row_const_off + k * SG::kKStr));
            const float offT = kk.x, offL = kk.y, cT = kk.z, cL = kk.w;
            float xv = 0.f, dtv = 0.f, dlv = 0.f;
            if constexpr (STAGE_X) {
              const T* xr = reinterpret_cast<const T*>(bufr + xd_off + k * kXK);
              xv = IO<T>::ld(xr); dtv = IO<T>::ld(xr + SG::kXTauBytes / sizeof(T)); dlv = IO<T>::ld(xr + 2 * SG::kXTauBytes / sizeof(T));
            } else if (ch_ok && ((bq.in_grid >> k) & 1u)) {
              const uint32_t off = cell_offq + (uint32_t)k * estep + (k >= bq.kw ? wrap_adj : 0u);
              xv = IO<T>::ld(reinterpret_cast<const T*>(Ximg + off));
              dtv = IO<T>::ld(reinterpret_cast<const T*>(DTimg + off));
              dlv = IO<T>::ld(reinterpret_cast<const T*>(DLimg + off));
            }
            uint32_t a_off = a_base_off;
            asm volatile("" : "+v"(a_off));
            const lds_float4* a_mine = (const lds_float4*)(uintptr_t)a_off;
            const char* rec = bufr + (rec_off + k * SG::kKStr);
            const float sT = __builtin_fmaf(cT * dtv, xv, g1);
            const float sL = cL * dlv * xv;
#pragma unroll
            for (int mg = 0; mg < 4; ++mg) {
              const v4f_t at4 = a_mine[mg], al4 = a_mine[kN / 4 + mg];
              const float4 b4 = *reinterpret_cast<const float4*>(rec + mg * SG::kPlane);
              const float4 l4 = *reinterpret_cast<const float4*>(rec + SG::kBLOff + mg * SG::kPlane);
              const float atq[4] = {at4.x, at4.y, at4.z, at4.w}, alq[4] = {al4.x, al4.y, al4.z, al4.w};
              const float bq4[4] = {b4.x, b4.y, b4.z, b4.w}, lq4[4] = {l4.x, l4.y, l4.z, l4.w};
              float aT[4], aL[4];   // gates before chains, see the forward kernel
#pragma unroll
              for (int qi = 0; qi < 4; ++qi) aT[qi] = fexp2(__builtin_fmaf(dtv, atq[qi], offT));
              pin4(aT);
              __builtin_amdgcn_sched_barrier(0);
#pragma unroll
              for (int qi = 0; qi < 4; ++qi) aL[qi] = fexp2(__builtin_fmaf(dlv, alq[qi], offL));
              pin4(aL);
              __builtin_amdgcn_sched_barrier(0);
#pragma unroll
              for (int qi = 0; qi < 4; ++qi) {
                float u = sL * lq4[qi];
                u = __builtin_fmaf(sT, bq4[qi], u);
                u = fma_row_below(aT[qi], hq[4 * mg + qi], u);
                hq[4 * mg + qi] = __builtin_fmaf(aL[qi], hq[4 * mg + qi], u);
              }
            }
          }
          typename Snap<ST>::quad* park = snapshot_of_lane(q + 1);   // the states before block q + 1
#pragma unroll
          for (int mg = 0; mg < 4; ++mg)
            if (ch_ok) park[snap_quad(mg)] = Snap<ST>::pack(hq[4 * mg], hq[4 * mg + 1], hq[4 * mg + 2], hq[4 * mg + 3]);   // (channels past E have no place of their own)
          __syncthreads();   // every wave is done with the buffer before the next block's copies land in it
        }
        if constexpr (!LATE_SNAPSHOT) load_ckpt(m, ck_take);
      }
      if constexpr (LATE_SNAPSHOT) load_ckpt(m, ck_take);
    }
    // the block before: where the lane's row will be is also what the lane's copies fetch
    const Pos Aprev = pos_before(A);
    const BlockPos bpn = block_pos(p, Aprev, rk, rbands);
    const int celln = cell_of(p, bpn.bnd0, r, bpn.col0);
    if constexpr (SWEEPS) ck_take = snapshot_lane(p, Pos{bpn.bnd0, bpn.col0}, r, ch_ok);
    if constexpr (STAGES) { if (direct) raw_copy_for(pos_before(Aprev), raw + rp * kRawBytes, m - 2 >= m_lo); }
    if (STAGES && m > m_lo) {
      if constexpr (SLICED) link.wait_for(link_need_bwd(m - 1 - m_lo, p.sl_nbb));
      if (direct) {
        stage_block<T, 4, CW, true, STAGE_X, NSTG, true>(p, lds + (cur ^ 1) * SG::kBytes, b, Aprev, bpn, celln, e_wg0, swave, lane, X, DT, DL, DY);
        bc_widen<SG, NSTG>(raw + (rp ^ 1) * kRawBytes, lds + (cur ^ 1) * SG::kBytes, swave, lane);
      } else {
        stage_block<T, 4, CW, true, STAGE_X, NSTG>(p, lds + (cur ^ 1) * SG::kBytes, b, Aprev, bpn, celln, e_wg0, swave, lane, X, DT, DL, DY);
      }
    }
    rp ^= 1;
    if constexpr (SWEEPS) cell_off0 = (uint32_t)(cell0 * p.E + e) * (uint32_t)sizeof(T);
    if constexpr (STAGES) f_off0 = (uint32_t)cell0 * (uint32_t)(3 * kN * sizeof(float)) + (BATCH ? (uint32_t)(slot * 4 * sizeof(float)) : f_sub);

    // The 16 states are swept in two halves of 8 (state groups 0,1 then 2,3), each half
    // recomputing and then back-propagating the whole block: only 5 x 8 recomputed states are
    // live at a time.  The state sums of the first half wait in `part4` for the second.
    float part4[kCK][4];
#pragma unroll
    for (int half = 0; half < 2; ++half) {
     if constexpr (!SWEEPS) {   // a wave that only stages: the barriers of a half, and its copies landed before the last one of the block
      if (BATCH && half == 1) { __syncthreads(); staging_landed(); }
     } else {
      float hb[kCK + 1][8];
      float gT_last[8], gL_last[8];   // gates of the last step: the adjoint starts with them
      if constexpr (BATCH) lead_if_younger<NW>(wave, true);   // (a barrier interval is a half: until the middle of its adjoint)
      // the states before the block: quad mg of the snapshot holds the states fold_state(mg, 0..3) in this order
      // (widened here, half by half: until then the snapshot stays as it came from memory)
      static_assert(sinv<PERM>(4 * 2 + 1) == fold_state(2, 1) && sinv<PERM>(4 * 3 + 2) == fold_state(3, 2), "snapshot quads are state groups");
#pragma unroll
      for (int mgl = 0; mgl < 2; ++mgl) {
        const float4 v = Snap<ST>::widen(cknext[2 * half + mgl]);
        hb[0][4 * mgl + 0] = v.x; hb[0][4 * mgl + 1] = v.y; hb[0][4 * mgl + 2] = v.z; hb[0][4 * mgl + 3] = v.w;
#pragma unroll
        for (int qi = 0; qi < 4; ++qi) { gT_last[4 * mgl + qi] = 0.f; gL_last[4 * mgl + qi] = 0.f; }
      }
      // ---- recompute the states of the block
#pragma unroll
      for (int k = 0; k < kCK; ++k) {
        const int t = t0 + k;
        if (t < p.T_total) {
          const float4 kk = *reinterpret_cast<const float4*>(bufc + (row_const_off + k * SG::kKStr));
          const float offT = kk.x, offL = kk.y, cT = kk.z, cL = kk.w;
          float xv = 0.f, dtv = 0.f, dlv = 0.f;
          if constexpr (STAGE_X) {
            const T* xr = reinterpret_cast<const T*>(bufc + xd_off + k * kXK);
            xv = IO<T>::ld(xr); dtv = IO<T>::ld(xr + SG::kXTauBytes / sizeof(T)); dlv = IO<T>::ld(xr + 2 * SG::kXTauBytes / sizeof(T));
          } else if (ch_ok && ((bp.in_grid >> k) & 1u)) {
            const uint32_t off = cell_off0 + (uint32_t)k * estep + (k >= bp.kw ? wrap_adj : 0u);
            xv = IO<T>::ld(reinterpret_cast<const T*>(Ximg + off));
            dtv = IO<T>::ld(reinterpret_cast<const T*>(DTimg + off));
            dlv = IO<T>::ld(reinterpret_cast<const T*>(DLimg + off));
          }
          // keep the per-step reads of A in LDS, not in live registers (the offset is hidden from
          // the optimiser; the pointer stays an LDS pointer so that the reads are ds_read)
          uint32_t a_off = a_base_off;
          asm volatile("" : "+v"(a_off));
          const lds_float4* a_mine = (const lds_float4*)(uintptr_t)a_off;
          const char* rec = bufc + (rec_off + k * SG::kKStr);
          const float sT = __builtin_fmaf(cT * dtv, xv, g1);
          const float sL = cL * dlv * xv;
#pragma unroll
          for (int mgl = 0; mgl < 2; ++mgl) {
            const int mg = 2 * half + mgl;
            const v4f_t at4 = a_mine[mg], al4 = a_mine[kN / 4 + mg];
            const float4 b4 = *reinterpret_cast<const float4*>(rec + mg * SG::kPlane);
            const float4 l4 = *reinterpret_cast<const float4*>(rec + SG::kBLOff + mg * SG::kPlane);
            const float atq[4] = {at4.x, at4.y, at4.z, at4.w}, alq[4] = {al4.x, al4.y, al4.z, al4.w};
            const float bq[4] = {b4.x, b4.y, b4.z, b4.w}, lq[4] = {l4.x, l4.y, l4.z, l4.w};
            float aT[4], aL[4];   // gates before chains, see the forward kernel
#pragma unroll
            for (int qi = 0; qi < 4; ++qi) aT[qi] = fexp2(__builtin_fmaf(dtv, atq[qi], offT));
            pin4(aT);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int qi = 0; qi < 4; ++qi) aL[qi] = fexp2(__builtin_fmaf(dlv, alq[qi], offL));
            pin4(aL);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int qi = 0; qi < 4; ++qi) {
              const int s8 = 4 * mgl + qi;
              float u = sL * lq[qi];
              u = __builtin_fmaf(sT, bq[qi], u);
              u = fma_row_below(aT[qi], hb[k][s8], u);
              hb[k + 1][s8] = __builtin_fmaf(aL[qi], hb[k][s8], u);
              if (k == kCK - 1) { gT_last[s8] = aT[qi]; gL_last[s8] = aL[qi]; }
            }
          }
        }
      }
      // ---- adjoint over the block, last step first
      if (BATCH && half == 1) __syncthreads();   // the sums of the first half have been taken out of the exchange buffers
#pragma unroll
      for (int k = kCK - 1; k >= 0; --k) {
        const int t = t0 + k;
        if (half == 1 && k == 0) staging_landed();   // before the last stores of the block, see the forward kernel
        if constexpr (BATCH) { if (k == 1) lead_if_younger<NW>(wave, false); }
        // the states of the later steps are dead by now: their registers take the next snapshot
        // (a longer checkpoint interval: not where the block before is the last of its group, whose state the replay will bring)
        if (!LATE_SNAPSHOT && half == 1 && k == (kCK > 1 ? 1 : 0) && m > m_lo && !opens_group(m - 1)) load_ckpt(m - 1, ck_take);
        if (t < p.T_total) {
          const float4 kk = *reinterpret_cast<const float4*>(bufc + (row_const_off + k * SG::kKStr));
          const float offT = kk.x, offL = kk.y, cT = kk.z, cL = kk.w;
          const bool inr = ch_ok && ((bp.in_grid >> k) & 1u);
          const uint32_t goff = cell_off0 + (uint32_t)k * estep + (k >= bp.kw ? wrap_adj : 0u);
          float xv = 0.f, dtv = 0.f, dlv = 0.f, dyv = 0.f;
          if constexpr (STAGE_X) {
            const T* xr = reinterpret_cast<const T*>(bufc + xd_off + k * kXK);
            xv = IO<T>::ld(xr); dtv = IO<T>::ld(xr + SG::kXTauBytes / sizeof(T)); dlv = IO<T>::ld(xr + 2 * SG::kXTauBytes / sizeof(T));
            dyv = IO<T>::ld(xr + 3 * SG::kXTauBytes / sizeof(T));
          } else if (inr) {
            xv = IO<T>::ld(reinterpret_cast<const T*>(Ximg + goff));
            dtv = IO<T>::ld(reinterpret_cast<const T*>(DTimg + goff));
            dlv = IO<T>::ld(reinterpret_cast<const T*>(DLimg + goff));
            dyv = IO<T>::ld(reinterpret_cast<const T*>(DYimg + goff));
          }
          uint32_t a_off = a_base_off;
          asm volatile("" : "+v"(a_off));
          const lds_float4* a_mine = (const lds_float4*)(uintptr_t)a_off;
          const char* rec = bufc + (rec_off + k * SG::kKStr);
          const float qT = cT * dtv * xv, qL = cL * dlv * xv;   // zero on lanes that are not grid cells
          const float dyl = dyv + gb1;
          float sT = 0.f, sL = 0.f, zT = 0.f, zL = 0.f;
          if (half == 1) { sT = part4[k][0]; sL = part4[k][1]; zT = part4[k][2]; zL = part4[k][3]; }
          float* sw = reinterpret_cast<float*>(slots + ((BATCH ? k : xpar) * NW + wave) * SLOT + lane);
          // A group of 4 states is folded over the 4 channel slots of the wave as soon as it is
          // done; afterwards the lane of slot q holds the channel sums of the states 4q..4q+3
          // (component mgl of its float2 after group mgl of this half).
#pragma unroll
          for (int mgl = 0; mgl < 2; ++mgl) {
            const int mg = 2 * half + mgl;
            const v4f_t at4 = a_mine[mg], al4 = a_mine[kN / 4 + mg];
            const float4 b4 = *reinterpret_cast<const float4*>(rec + mg * SG::kPlane);
            const float4 l4 = *reinterpret_cast<const float4*>(rec + SG::kBLOff + mg * SG::kPlane);
            const float4 c4 = *reinterpret_cast<const float4*>(rec + SG::kCOff + mg * SG::kPlane);
            const float atq[4] = {at4.x, at4.y, at4.z, at4.w}, alq[4] = {al4.x, al4.y, al4.z, al4.w};
            const float bq[4] = {b4.x, b4.y, b4.z, b4.w}, lq[4] = {l4.x, l4.y, l4.z, l4.w}, cq[4] = {c4.x, c4.y, c4.z, c4.w};
            float vC[4], vBT[4], vBL[4];
#pragma unroll
            for (int qi = 0; qi < 4; ++qi) {
              const int n = fold_state(mg, qi), s8 = 4 * mgl + qi;
              const float a2t = atq[qi], a2l = alq[qi];
              const float aT = k == kCK - 1 ? gT_last[s8] : fexp2(__builtin_fmaf(dtv, a2t, offT));
              const float aL = k == kCK - 1 ? gL_last[s8] : fexp2(__builtin_fmaf(dlv, a2l, offL));
              const float lam = __builtin_fmaf(dyl, cq[qi], add_row_above(muL[n], muT[n]));
              const float mT = aT * lam, mL = aL * lam;
              muT[n] = mT;
              muL[n] = mL;
              const float ZT = mul_row_below(mT, hb[k][s8]), ZL = mL * hb[k][s8];
              accAT[n] = __builtin_fmaf(ZT, dtv, accAT[n]);
              accAL[n] = __builtin_fmaf(ZL, dlv, accAL[n]);
              zT = __builtin_fmaf(ZT, a2t, zT);
              zL = __builtin_fmaf(ZL, a2l, zL);
              sT = __builtin_fmaf(lam, bq[qi], sT);
              sL = __builtin_fmaf(lam, lq[qi], sL);
              vBT[qi] = qT * lam;
              vBL[qi] = qL * lam;
              vC[qi] = dyv * hb[k + 1][s8];
            }
            sw[mgl] = fold16(fold32(vC[0], vC[1]), fold32(vC[2], vC[3]));
            sw[64 * 2 + mgl] = fold16(fold32(vBT[0], vBT[1]), fold32(vBT[2], vBT[3]));
            sw[128 * 2 + mgl] = fold16(fold32(vBL[0], vBL[1]), fold32(vBL[2], vBL[3]));
          }
          if (p.nbands > 1 && !p.stacked) {   // first row of a band: the lower ghost of the band above will replay its muT
            const bool wk = k >= bp.kw;
            if (inr && r == 1 && (wk ? bp.bnd0 + 1 : bp.bnd0) >= 1) {
              const int ck = wk ? bp.col0 + k - p.S : bp.col0 + k;
              char* bb = BOTimg + (wk ? bp.bnd0 + 1 : bp.bnd0) * p.bot_stride * (int64_t)sizeof(float) +
                         (uint32_t)(ck * p.E + e) * (uint32_t)(kN * sizeof(float));
#pragma unroll
              for (int q = 2 * half; q < 2 * half + 2; ++q) {   // the two state groups of this half, as of this step
                const float4 row = make_float4(muT[sinv<PERM>(4 * q)], muT[sinv<PERM>(4 * q + 1)], muT[sinv<PERM>(4 * q + 2)], muT[sinv<PERM>(4 * q + 3)]);
                if constexpr (SLICED) store_row_device_scope(reinterpret_cast<float4*>(bb) + q, row); else reinterpret_cast<float4*>(bb)[q] = row;
              }
            }
          }
          if (half == 0) {
            part4[k][0] = sT; part4[k][1] = sL; part4[k][2] = zT; part4[k][3] = zL;
          } else {
            accD = __builtin_fmaf(dyv, xv, accD);
            if (inr) {
              float gdT = __builtin_fmaf(cT * xv, sT, kLn2 * zT), gdL = __builtin_fmaf(cL * xv, sL, kLn2 * zL);
              if (p.dpre) {   // (uniform) gradients with respect to what the softplus was applied to
                gdT *= softplus_slope<T>(dtv);
                gdL *= softplus_slope<T>(dlv);
              }
              IO<T>::st(reinterpret_cast<T*>(DDTimg + goff), gdT);
              IO<T>::st(reinterpret_cast<T*>(DDLimg + goff), gdL);
              IO<T>::st(reinterpret_cast<T*>(DXimg + goff), __builtin_fmaf(cT * dtv, sT, __builtin_fmaf(cL * dlv, sL, dyv * dsk)));
            }
          }
          // ---- across the waves of the workgroup: the per-wave slots (this half's two state
          // groups) are added in wave order, one sum per thread, the same share for every wave
          if constexpr (!BATCH) {
            __syncthreads();
            if (f_on && ((bp.in_grid >> k) & 1u)) {
              const uint32_t off = f_off0 + (uint32_t)k * pstep + (k >= bp.kw ? pwrap_adj : 0u) + (uint32_t)(2 * half * sizeof(float));
              if constexpr (PAIRS) {
                const float2* sl = slots + xpar * NW * SLOT + f_it;
                float2 s = sl[0];
#pragma unroll
                for (int w = 1; w < NW; ++w) { s.x += sl[w * SLOT].x; s.y += sl[w * SLOT].y; }
                *reinterpret_cast<float2*>(PARTimg + off) = s;
              } else {
                const float* sl = reinterpret_cast<const float*>(slots + xpar * NW * SLOT + f_it) + f_comp;
                float s = sl[0];
#pragma unroll
                for (int w = 1; w < NW; ++w) s += sl[2 * w * SLOT];
                *reinterpret_cast<float*>(PARTimg + off) = s;
              }
            }
            xpar ^= 1;
          }
        }
      }
     }
      if constexpr (BATCH) {
        // ---- across the waves, all steps of this half at once: the kCK x 3 (step, tensor) sets of
        // sums are dealt to the waves; a thread adds up the float2 of the lane (its slot, its row)
        __syncthreads();
        if constexpr (STAGES)
#pragma unroll
        for (int rd = 0; rd < (kCK * 3 + NSTG - 1) / NSTG; ++rd) {
          const int j = rd * NSTG + swave;                 // (uniform)
          if (j < kCK * 3) {
            const int k = j / 3, v = j - 3 * k;
            if ((bp.in_grid >> k) & 1u) {
              const uint32_t off = f_off0 + (uint32_t)k * pstep + (k >= bp.kw ? pwrap_adj : 0u) + (uint32_t)((v * kN + 2 * half) * sizeof(float));
              const float2* sl = slots + k * NW * SLOT + v * 64 + lane;
              float2 sum = sl[0];
#pragma unroll
              for (int w = 1; w < NW; ++w) { sum.x += sl[w * SLOT].x; sum.y += sl[w * SLOT].y; }
              *reinterpret_cast<float2*>(PARTimg + off) = sum;
            }
          }
        }
      }
    }
    __syncthreads();
    // Every wave has waited, before the last adjoint step of this block, for all it had issued: the blocks swept
    // before this one are in memory, and so are the rows this block stored in its steps 3, 2 and 1.  The band above
    // needs, of the newest block it is told about, the steps 3 and 2 only (link_need_bwd), so this block counts.
    if constexpr (SLICED && STAGES) link.publish((uint32_t)(m_hi - m));
    A = Aprev;
    bp = bpn;
    cell0 = celln;
    cur ^= 1;
  }
  };
  if constexpr (NH == 0) sweep(std::integral_constant<int, kAll>{});
  else if (helper) sweep(std::integral_constant<int, kStager>{});
  else sweep(std::integral_constant<int, kSweeper>{});
  bool broken = false;
  if constexpr (SLICED) {   // the whole window is done once every store of every wave has completed
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    link.publish((uint32_t)p.sl_nbb);
    broken = link.broken() || link_poll(p.link_err) != 0u;   // (also a workgroup of the forward sweep that rebuilt the snapshots for this launch)
    if constexpr (NH > 0) {   // only the waves that wait know of a wait given up: they tell the others (the staging buffers are free now)
      if ((int)threadIdx.x == link.pub) *reinterpret_cast<volatile uint32_t*>(lds) = link.broken() ? 1u : 0u;
      __syncthreads();
      broken = broken || *reinterpret_cast<volatile uint32_t*>(lds) != 0u;
    }
    if (broken) poison_band<T>(p, my_band, b, e_wg0, CW, p.dx, p.ddT, p.ddL);
  }

  // ---- sums over positions: reduce over the rows of the band (lanes of one channel slot)
  float red[2 * kN + 1];
#pragma unroll
  for (int n = 0; n < kN; ++n) { red[n] = accAT[n]; red[kN + n] = accAL[n]; }
  red[2 * kN] = broken ? __builtin_nanf("") : accD;
  if (broken) { red[0] = __builtin_nanf(""); red[kN] = __builtin_nanf(""); }   // (d_AT, d_AL, d_D of the channel say so too)
#pragma unroll
  for (int k = 0; k < 2 * kN + 1; ++k) {
    float v = red[k];
#pragma unroll
    for (int off = kHB >> 1; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    red[k] = v;
  }
  if (ch_ok && r == 0) {
    const int64_t slot_e = ((int64_t)b * p.pa_slots + (SLICED ? my_band : 0)) * p.E + e;
    float* pa = p.pA + slot_e * (2 * kN);
#pragma unroll
    for (int n = 0; n < 2 * kN; ++n) pa[n] = red[n];
    p.pD[slot_e] = red[2 * kN];
  }
}

// --------------------------------------------------- backward from snapshots every 2 steps
// The same adjoint as m2d_bwd_kernel for a forward that kept the state before the steps 0 and 2 of every block
// (and the state behind the last block): the kernel is out of instruction issue slots long before it is out of
// memory bandwidth, so it reads twice the snapshots and recomputes one step in two instead of all four, and
// computes the gates of every step once instead of 1.75 times.  A block is swept as two sub-blocks of 2 steps,
// each in two halves of 8 states (the registers of a lane hold no more): restore the state before the sub-block,
// recompute the state between its two steps keeping that step's gates, take the state behind the sub-block from
// the snapshot after it, and run the adjoint over the two steps.  The snapshot quads of a half-pass are fetched
// while the half-pass before is worked on.  Channel sums cross the waves through two exchange sets per half of
// the states, used alternately by the half-passes: one barrier per half-pass, and the sums of one half are added
// up while the other half is computed.
// Schedules: one stream per image, or stacked images (not the linked sweep, whose problems are few large images
// where the snapshots weigh most).
template <typename T, int NW>
constexpr int bwd2_exchange_sets() {   // sets of [wave][3][64] float2: 2 halves x 2 steps where they fit, else 2 used alternately per step
  return sizeof(float2) * 4 * NW * 3 * 64 + sizeof(float) * NW * 4 * 2 * kN + 256 +
         2 * (size_t)Stage<T, 4, NW * 4, true>::kBytes + (sizeof(T) == 2 ? 2 * kRawBytes : 0) <= 160 * 1024 ? 4 : 2;
}
template <typename T, bool STAGE_X, int MODE, int NW = kBwdWaves>
__global__ __launch_bounds__((NW + whole_helpers<MODE, NW>()) * 64) void m2d_bwd2_kernel(const ScanParams pin) {
  static_assert(MODE != kModeSliced, "the linked sweep keeps a snapshot every 4 steps");
  constexpr bool STACKED = MODE == kModeStacked;
  ScanParams p = pin;   // (stacked images: the height is shortened below for a last, shorter stack)
  if constexpr (!STACKED) {
    __builtin_assume(p.stacked == 0);
    __builtin_assume(p.rb == kRB);
    __builtin_assume(p.S >= kHB + kCK - 1);
  }
  static_assert(kCK == 4, "two sub-blocks of 2 steps");
  constexpr int CS = 64 >> kHBShift;     // 4 channel slots
  constexpr int SLOT = 3 * 64;           // float2s per wave in one exchange set
  constexpr int CW = NW * CS;
  constexpr bool PERM = true;
  constexpr int NH = whole_helpers<MODE, NW>();   // waves that only stage and add up the channel sums (then the first NW waves only sweep)
  constexpr int NSTG = NH ? NH : NW;              // waves that share the copies of a block and the sums of a half-pass
  using SG = Stage<T, 4, CW, true>;
  extern __shared__ float4 smem[];
  constexpr int XSETS = bwd2_exchange_sets<T, NW>();
  constexpr bool BATCH = XSETS == 4;
  static_assert(NH == 0 || BATCH, "the waves that stage add up the sums of a half-pass in one go");
  float2* slots = reinterpret_cast<float2*>(smem);                       // BATCH: [half][step of the sub-block][wave][3][64], else [2][wave][3][64]
  float* a_lds = reinterpret_cast<float*>(slots + XSETS * NW * SLOT);    // [wave][CS][2][16], fold order
  char* lds = reinterpret_cast<char*>(a_lds + NW * CS * 2 * kN);         // 2 staging buffers
  constexpr bool WIDEN = sizeof(T) == 2;
  char* raw = lds + 2 * SG::kBytes;         // [2][kRawBytes]: 16-bit B_T, B_L, C on their way
  const bool direct = WIDEN && p.bc_direct != 0;   // (uniform)
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lb = logical_block(p.nwg);
  const int m_hi = p.nblk;
  const int b = lb / p.bpb;
  const int eg = lb % p.bpb;
  if constexpr (STACKED) {   // the last stack of the batch may hold fewer images
    const int nimg = p.Breal - b * p.ips < p.ips ? p.Breal - b * p.ips : p.ips;
    p.H = nimg * p.Himg;
    p.nbands = (p.H + p.rb - 1) / p.rb;
    p.rows_last = p.H - (p.nbands - 1) * p.rb;
  }
  const int e_wg0 = eg * CW;
  const bool helper = NH && wave >= NW;      // (uniform) stages and adds up, never sweeps
  const bool stages = !NH || helper;
  const int swave = NH ? wave - NW : wave;   // the wave's turn among those that stage
  const int slot = lane >> kHBShift, r = lane & (kHB - 1);
  const int rbands = row_bands(p, r);
  const int rk = STACKED ? skew_row(p, r) : r;
  const int ch_loc = (helper ? swave : wave) * CS + slot;
  const int e_raw = e_wg0 + ch_loc;
  const bool ch_ok = !helper && e_raw < p.E;
  const int e = e_raw < p.E ? e_raw : p.E - 1;
  if (!helper) {  // A of the wave's channels into LDS in fold order (read back group by group)
    float* mine = a_lds + ch_loc * (2 * kN);
    mine[spos<true>(r)] = p.A2T[e * kN + r];
    mine[kN + spos<true>(r)] = p.A2L[e * kN + r];
  }
  for (int i = threadIdx.x; i < 2 * SG::kBytes / 16; i += (NW + NH) * 64) reinterpret_cast<float4*>(lds)[i] = make_float4(0.f, 0.f, 0.f, 0.f);
  const uint32_t a_base_off = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) float*)(a_lds + ch_loc * (2 * kN)));
  const float dsk = p.Df[e];
  settle_loads();

  const T* X = static_cast<const T*>(p.x);
  const T* DT = static_cast<const T*>(p.dT);
  const T* DL = static_cast<const T*>(p.dL);
  const T* DY = static_cast<const T*>(p.dy);
  const int64_t img_cell0 = (int64_t)b * p.Hs * p.W;
  const int64_t img_bytes = img_cell0 * p.E * (int64_t)sizeof(T);
  const char* Ximg = reinterpret_cast<const char*>(X) + img_bytes;
  const char* DTimg = reinterpret_cast<const char*>(DT) + img_bytes;
  const char* DLimg = reinterpret_cast<const char*>(DL) + img_bytes;
  const char* DYimg = reinterpret_cast<const char*>(DY) + img_bytes;
  char* DXimg = static_cast<char*>(p.dx) + img_bytes;
  char* DDTimg = static_cast<char*>(p.ddT) + img_bytes;
  char* DDLimg = static_cast<char*>(p.ddL) + img_bytes;
  char* BOTimg = reinterpret_cast<char*>(p.bot + (int64_t)b * p.W * p.E * kN);
  char* PARTimg = reinterpret_cast<char*>(p.part + ((int64_t)eg * p.Ptot + img_cell0) * (3 * kN));

  float accAT[kN], accAL[kN], accD = 0.f;
  float muT[kN], muL[kN];
#pragma unroll
  for (int n = 0; n < kN; ++n) { accAT[n] = 0.f; accAL[n] = 0.f; muT[n] = 0.f; muL[n] = 0.f; }
  const uint32_t rec_off = STACKED ? r * 16 : (r == 0 ? SG::top_off(ch_loc) : (r == kHB - 1 ? SG::bot_off(ch_loc) - SG::kCOff : r * 16));
  const uint32_t xd_off = SG::kXOff + SG::x_off(r, ch_loc);
  constexpr uint32_t kXK = SG::kXStepBytes;
  // the sum that this thread adds up in the exchange: see m2d_bwd_kernel
  constexpr bool PAIRS = NW * 64 < 2 * SLOT;
  const int f_combo = wave * 4 + slot;
  const bool f_on = f_combo < (PAIRS ? 12 : 24);
  const int f_v = PAIRS ? f_combo >> 2 : f_combo >> 3, f_s = PAIRS ? f_combo & 3 : (f_combo >> 1) & 3;
  const int f_comp = PAIRS ? 0 : f_combo & 1;
  const int f_it = f_v * 64 + f_s * kHB + r;
  const uint32_t f_sub = (uint32_t)(f_v * kN + f_s * 4 + f_comp) * (uint32_t)sizeof(float);
  const float g1 = !STACKED && r == 0 ? 1.f : 0.f;
  const float gb1 = !STACKED && r == kHB - 1 ? 1.f : 0.f;
  const uint32_t estep = (uint32_t)(p.flip ? -p.E : p.E) * (uint32_t)sizeof(T);
  const uint32_t wrap_adj = (uint32_t)(p.rb * p.W - p.S) * estep;
  const uint32_t pstep = (uint32_t)(p.flip ? -1 : 1) * (uint32_t)(3 * kN * sizeof(float));
  const uint32_t pwrap_adj = (uint32_t)(p.rb * p.W - p.S) * pstep;
  const uint32_t row_const_off = SG::kConstPlane * SG::kPlane + r * 16;

  BlockPos bp;
  uint32_t cell_off0 = 0, f_off0 = 0;
  typedef typename Snap<T>::quad quad_t;
  // The two quads (8 states) of snapshot `idx` that half `hf` of the states works on, as they come from memory
  // (take: the forward left the lane's own state there, see snapshot_lane; snapshot 0 is the state before the sweep).
  auto load_snap = [&](quad_t (&dst)[2], int idx, int hf, bool take) {
    if (idx == 0 || !take) {
      dst[0] = Snap<T>::zero(); dst[1] = Snap<T>::zero();
    } else {
      Snap<T>::load2(snapshot_at<T>(p, b, idx, e, p.ck_nblk) + snap_lane(r) + snap_quad(2 * hf), dst);
    }
  };
  auto widen8 = [&](const quad_t (&src)[2], float (&dst)[8]) {
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const float4 v = Snap<T>::widen(src[q]);
      dst[4 * q + 0] = v.x; dst[4 * q + 1] = v.y; dst[4 * q + 2] = v.z; dst[4 * q + 3] = v.w;
    }
  };
  auto pos_at = [&](const BlockPos& q, int k) {   // the row's position at step k of the block (k <= kCK: one band change at most)
    Pos o;
    const bool w = k >= q.kw;
    o.bnd = w ? q.bnd0 + 1 : q.bnd0;
    o.col = w ? k - q.kw : q.col0 + k;
    return o;
  };
  auto pos_before = [&](Pos Q) {
    Q.col -= kCK;
    if (Q.col < 0) { Q.col += p.S; Q.bnd -= 1; }
    return Q;
  };

  Pos A = pos_of(p, (m_hi - 1) * kCK - (kHB - 1));
  __syncthreads();   // the zeros are in place before the first copies land on them
  bp = block_pos(p, A, rk, rbands);
  int cell0 = cell_of(p, bp.bnd0, r, bp.col0);
  // take[s]: whether the lane restores snapshot 2m + s of the block being swept (the states before its steps 0 and
  // 2 and behind its step 3)
  bool take0 = snapshot_lane(p, Pos{bp.bnd0, bp.col0}, r, ch_ok), take1 = snapshot_lane(p, pos_at(bp, 2), r, ch_ok);
  const bool take2 = snapshot_lane(p, pos_at(bp, kCK), r, ch_ok);
  // Snapshot quads on their way, per half of the states: qa[half] the state before the sub-block that the half's next
  // half-pass sweeps (fetched two half-passes ahead: when the half's pass before starts), qn[half] the state behind
  // that sub-block, which is the state before the sub-block that the half swept last (its qa, kept as it came).
  quad_t qa[2][2], qn[2][2];
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    load_snap(qa[hf], 2 * (m_hi - 1) + 1, hf, take1);
    load_snap(qn[hf], 2 * (m_hi - 1) + 2, hf, take2);
  }
  auto raw_copy_for = [&](Pos A2, char* dst, bool live) {
    const BlockPos q2 = block_pos(p, A2, rk, rbands);
    bc_raw_copy<NSTG>(p, pin.bcd, dst, b, q2, cell_of(p, q2.bnd0, r, q2.col0), swave, lane, live);
  };
  int rp = 0;
  if (direct) {
    if (stages) bc_raw_copy<NSTG>(p, pin.bcd, raw, b, bp, cell0, swave, lane, true);
    if (stages) raw_copy_for(pos_before(A), raw + kRawBytes, m_hi - 2 >= 0);
    if (stages) stage_block<T, 4, CW, true, STAGE_X, NSTG, true>(p, lds, b, A, bp, cell0, e_wg0, swave, lane, X, DT, DL, DY);
    staging_fence();
    if (stages) bc_widen<SG, NSTG>(raw, lds, swave, lane);
  } else {
    if (stages) stage_block<T, 4, CW, true, STAGE_X, NSTG>(p, lds, b, A, bp, cell0, e_wg0, swave, lane, X, DT, DL, DY);
  }
  staging_fence();
  int cur = 0;
  int xpar = 0;   // (one set per step: the exchange set in use)

  // The sweep over the blocks, as a wave of the given role runs it (see m2d_fwd_kernel).
  auto sweep = [&](auto role) {
  constexpr int ROLE = decltype(role)::value;
  constexpr bool STAGES = ROLE != kSweeper, SWEEPS = ROLE != kStager;
  for (int m = m_hi - 1; m >= 0; --m) {
    const int t0 = m * kCK;
    const char* bufc = lds + cur * SG::kBytes;
    const Pos Aprev = pos_before(A);
    const BlockPos bpn = block_pos(p, Aprev, rk, rbands);
    const int celln = cell_of(p, bpn.bnd0, r, bpn.col0);
    bool take0n = false, take1n = false;
    if constexpr (SWEEPS) { take0n = snapshot_lane(p, Pos{bpn.bnd0, bpn.col0}, r, ch_ok); take1n = snapshot_lane(p, pos_at(bpn, 2), r, ch_ok); }
    if constexpr (STAGES) { if (direct) raw_copy_for(pos_before(Aprev), raw + rp * kRawBytes, m - 2 >= 0); }
    if (STAGES && m > 0) {
      if (direct) {
        stage_block<T, 4, CW, true, STAGE_X, NSTG, true>(p, lds + (cur ^ 1) * SG::kBytes, b, Aprev, bpn, celln, e_wg0, swave, lane, X, DT, DL, DY);
        bc_widen<SG, NSTG>(raw + (rp ^ 1) * kRawBytes, lds + (cur ^ 1) * SG::kBytes, swave, lane);
      } else {
        stage_block<T, 4, CW, true, STAGE_X, NSTG>(p, lds + (cur ^ 1) * SG::kBytes, b, Aprev, bpn, celln, e_wg0, swave, lane, X, DT, DL, DY);
      }
    }
    rp ^= 1;
    if constexpr (SWEEPS) cell_off0 = (uint32_t)(cell0 * p.E + e) * (uint32_t)sizeof(T);
    if constexpr (STAGES) f_off0 = (uint32_t)cell0 * (uint32_t)(3 * kN * sizeof(float)) + (BATCH ? (uint32_t)(slot * 4 * sizeof(float)) : f_sub);

#pragma unroll
    for (int sub = 1; sub >= 0; --sub) {
      const int k0 = 2 * sub;
      float part2[2][4];   // the state sums of the first half wait here for the second
#pragma unroll
      for (int half = 0; half < 2; ++half) {
       if constexpr (!SWEEPS) {   // a wave that only stages: its copies have landed before the barrier that ends the block
        if (sub == 0 && half == 1) staging_landed();
       } else {
        float ha[8], hb1[8], hn[8], gT[8], gL[8];
        lead_if_younger<NW>(wave, true);    // (until the second step of the adjoint below)
        widen8(qa[half], ha);
        widen8(qn[half], hn);
        qn[half][0] = qa[half][0]; qn[half][1] = qa[half][1];
        // the quads of this half's next pass (the first sub-block's passes fetch behind this block's copies for the
        // second sub-block, the second's for the block to come, in time for that block's wait for everything in flight)
        if (sub == 1) load_snap(qa[half], 2 * m, half, take0);
        else if (m > 0) load_snap(qa[half], 2 * (m - 1) + 1, half, take1n);
        // ---- recompute the state between the two steps
        if (t0 + k0 < p.T_total) {
          const int k = k0;
          const float4 kk = *reinterpret_cast<const float4*>(bufc + (row_const_off + k * SG::kKStr));
          const float offT = kk.x, offL = kk.y, cT = kk.z, cL = kk.w;
          float xv = 0.f, dtv = 0.f, dlv = 0.f;
          if constexpr (STAGE_X) {
            const T* xr = reinterpret_cast<const T*>(bufc + xd_off + k * kXK);
            xv = IO<T>::ld(xr); dtv = IO<T>::ld(xr + SG::kXTauBytes / sizeof(T)); dlv = IO<T>::ld(xr + 2 * SG::kXTauBytes / sizeof(T));
          } else if (ch_ok && ((bp.in_grid >> k) & 1u)) {
            const uint32_t off = cell_off0 + (uint32_t)k * estep + (k >= bp.kw ? wrap_adj : 0u);
            xv = IO<T>::ld(reinterpret_cast<const T*>(Ximg + off));
            dtv = IO<T>::ld(reinterpret_cast<const T*>(DTimg + off));
            dlv = IO<T>::ld(reinterpret_cast<const T*>(DLimg + off));
          }
          uint32_t a_off = a_base_off;
          asm volatile("" : "+v"(a_off));
          const lds_float4* a_mine = (const lds_float4*)(uintptr_t)a_off;
          const char* rec = bufc + (rec_off + k * SG::kKStr);
          const float sT = __builtin_fmaf(cT * dtv, xv, g1);
          const float sL = cL * dlv * xv;
#pragma unroll
          for (int mgl = 0; mgl < 2; ++mgl) {
            const int mg = 2 * half + mgl;
            const v4f_t at4 = a_mine[mg], al4 = a_mine[kN / 4 + mg];
            const float4 b4 = *reinterpret_cast<const float4*>(rec + mg * SG::kPlane);
            const float4 l4 = *reinterpret_cast<const float4*>(rec + SG::kBLOff + mg * SG::kPlane);
            const float atq[4] = {at4.x, at4.y, at4.z, at4.w}, alq[4] = {al4.x, al4.y, al4.z, al4.w};
            const float bq[4] = {b4.x, b4.y, b4.z, b4.w}, lq[4] = {l4.x, l4.y, l4.z, l4.w};
            float aT[4], aL[4];   // gates before chains, see the forward kernel
#pragma unroll
            for (int qi = 0; qi < 4; ++qi) aT[qi] = fexp2(__builtin_fmaf(dtv, atq[qi], offT));
            pin4(aT);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int qi = 0; qi < 4; ++qi) aL[qi] = fexp2(__builtin_fmaf(dlv, alq[qi], offL));
            pin4(aL);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int qi = 0; qi < 4; ++qi) {
              const int s8 = 4 * mgl + qi;
              float u = sL * lq[qi];
              u = __builtin_fmaf(sT, bq[qi], u);
              u = fma_row_below(aT[qi], ha[s8], u);
              hb1[s8] = __builtin_fmaf(aL[qi], ha[s8], u);
              gT[s8] = aT[qi]; gL[s8] = aL[qi];
            }
          }
        }
        // ---- adjoint over the sub-block, second step first
#pragma unroll
        for (int ks = 1; ks >= 0; --ks) {
          const int k = k0 + ks;
          const int t = t0 + k;
          if (ks == 0) lead_if_younger<NW>(wave, false);
          if (sub == 0 && half == 1 && ks == 0) staging_landed();   // before the last stores of the block, see the forward kernel
          if (t < p.T_total) {
            const float (&hbk)[8] = ks == 1 ? hb1 : ha;    // the state before this step
            const float (&hnk)[8] = ks == 1 ? hn : hb1;    // ... and behind it
            const float4 kk = *reinterpret_cast<const float4*>(bufc + (row_const_off + k * SG::kKStr));
            const float offT = kk.x, offL = kk.y, cT = kk.z, cL = kk.w;
            const bool inr = ch_ok && ((bp.in_grid >> k) & 1u);
            const uint32_t goff = cell_off0 + (uint32_t)k * estep + (k >= bp.kw ? wrap_adj : 0u);
            float xv = 0.f, dtv = 0.f, dlv = 0.f, dyv = 0.f;
            if constexpr (STAGE_X) {
              const T* xr = reinterpret_cast<const T*>(bufc + xd_off + k * kXK);
              xv = IO<T>::ld(xr); dtv = IO<T>::ld(xr + SG::kXTauBytes / sizeof(T)); dlv = IO<T>::ld(xr + 2 * SG::kXTauBytes / sizeof(T));
              dyv = IO<T>::ld(xr + 3 * SG::kXTauBytes / sizeof(T));
            } else if (inr) {
              xv = IO<T>::ld(reinterpret_cast<const T*>(Ximg + goff));
              dtv = IO<T>::ld(reinterpret_cast<const T*>(DTimg + goff));
              dlv = IO<T>::ld(reinterpret_cast<const T*>(DLimg + goff));
              dyv = IO<T>::ld(reinterpret_cast<const T*>(DYimg + goff));
            }
            uint32_t a_off = a_base_off;
            asm volatile("" : "+v"(a_off));
            const lds_float4* a_mine = (const lds_float4*)(uintptr_t)a_off;
            const char* rec = bufc + (rec_off + k * SG::kKStr);
            const float qT = cT * dtv * xv, qL = cL * dlv * xv;   // zero on lanes that are not grid cells
            const float dyl = dyv + gb1;
            float sT = 0.f, sL = 0.f, zT = 0.f, zL = 0.f;
            if (half == 1) { sT = part2[ks][0]; sL = part2[ks][1]; zT = part2[ks][2]; zL = part2[ks][3]; }
            float* sw = reinterpret_cast<float*>(slots + ((BATCH ? 2 * half + ks : xpar) * NW + wave) * SLOT + lane);
#pragma unroll
            for (int mgl = 0; mgl < 2; ++mgl) {
              const int mg = 2 * half + mgl;
              const v4f_t at4 = a_mine[mg], al4 = a_mine[kN / 4 + mg];
              const float4 b4 = *reinterpret_cast<const float4*>(rec + mg * SG::kPlane);
              const float4 l4 = *reinterpret_cast<const float4*>(rec + SG::kBLOff + mg * SG::kPlane);
              const float4 c4 = *reinterpret_cast<const float4*>(rec + SG::kCOff + mg * SG::kPlane);
              const float atq[4] = {at4.x, at4.y, at4.z, at4.w}, alq[4] = {al4.x, al4.y, al4.z, al4.w};
              const float bq[4] = {b4.x, b4.y, b4.z, b4.w}, lq[4] = {l4.x, l4.y, l4.z, l4.w}, cq[4] = {c4.x, c4.y, c4.z, c4.w};
              float vC[4], vBT[4], vBL[4];
#pragma unroll
              for (int qi = 0; qi < 4; ++qi) {
                const int n = fold_state(mg, qi), s8 = 4 * mgl + qi;
                const float a2t = atq[qi], a2l = alq[qi];
                const float aT = ks == 0 ? gT[s8] : fexp2(__builtin_fmaf(dtv, a2t, offT));
                const float aL = ks == 0 ? gL[s8] : fexp2(__builtin_fmaf(dlv, a2l, offL));
                const float lam = __builtin_fmaf(dyl, cq[qi], add_row_above(muL[n], muT[n]));
                const float mT = aT * lam, mL = aL * lam;
                muT[n] = mT;
                muL[n] = mL;
                const float ZT = mul_row_below(mT, hbk[s8]), ZL = mL * hbk[s8];
                accAT[n] = __builtin_fmaf(ZT, dtv, accAT[n]);
                accAL[n] = __builtin_fmaf(ZL, dlv, accAL[n]);
                zT = __builtin_fmaf(ZT, a2t, zT);
                zL = __builtin_fmaf(ZL, a2l, zL);
                sT = __builtin_fmaf(lam, bq[qi], sT);
                sL = __builtin_fmaf(lam, lq[qi], sL);
                vBT[qi] = qT * lam;
                vBL[qi] = qL * lam;
                vC[qi] = dyv * hnk[s8];
              }
              sw[mgl] = fold16(fold32(vC[0], vC[1]), fold32(vC[2], vC[3]));
              sw[64 * 2 + mgl] = fold16(fold32(vBT[0], vBT[1]), fold32(vBT[2], vBT[3]));
              sw[128 * 2 + mgl] = fold16(fold32(vBL[0], vBL[1]), fold32(vBL[2], vBL[3]));
            }
            if (p.nbands > 1 && !p.stacked) {   // first row of a band: the lower ghost of the band above will replay its muT
              const bool wk = k >= bp.kw;
              if (inr && r == 1 && (wk ? bp.bnd0 + 1 : bp.bnd0) >= 1) {
                const int ck = wk ? bp.col0 + k - p.S : bp.col0 + k;
                char* bb = BOTimg + (wk ? bp.bnd0 + 1 : bp.bnd0) * p.bot_stride * (int64_t)sizeof(float) +
                           (uint32_t)(ck * p.E + e) * (uint32_t)(kN * sizeof(float));
#pragma unroll
                for (int q = 2 * half; q < 2 * half + 2; ++q)
                  reinterpret_cast<float4*>(bb)[q] = make_float4(muT[sinv<PERM>(4 * q)], muT[sinv<PERM>(4 * q + 1)], muT[sinv<PERM>(4 * q + 2)], muT[sinv<PERM>(4 * q + 3)]);
              }
            }
            if (half == 0) {
              part2[ks][0] = sT; part2[ks][1] = sL; part2[ks][2] = zT; part2[ks][3] = zL;
            } else {
              accD = __builtin_fmaf(dyv, xv, accD);
              if (inr) {
                float gdT = __builtin_fmaf(cT * xv, sT, kLn2 * zT), gdL = __builtin_fmaf(cL * xv, sL, kLn2 * zL);
                if (p.dpre) {   // (uniform) gradients with respect to what the softplus was applied to
                  gdT *= softplus_slope<T>(dtv);
                  gdL *= softplus_slope<T>(dlv);
                }
                IO<T>::st(reinterpret_cast<T*>(DDTimg + goff), gdT);
                IO<T>::st(reinterpret_cast<T*>(DDLimg + goff), gdL);
                IO<T>::st(reinterpret_cast<T*>(DXimg + goff), __builtin_fmaf(cT * dtv, sT, __builtin_fmaf(cL * dlv, sL, dyv * dsk)));
              }
            }
            if constexpr (!BATCH) {   // ---- across the waves, this step: as in m2d_bwd_kernel
              __syncthreads();
              if (f_on && ((bp.in_grid >> k) & 1u)) {
                const uint32_t off = f_off0 + (uint32_t)k * pstep + (k >= bp.kw ? pwrap_adj : 0u) + (uint32_t)(2 * half * sizeof(float));
                if constexpr (PAIRS) {
                  const float2* sl = slots + xpar * NW * SLOT + f_it;
                  float2 s = sl[0];
#pragma unroll
                  for (int w = 1; w < NW; ++w) { s.x += sl[w * SLOT].x; s.y += sl[w * SLOT].y; }
                  *reinterpret_cast<float2*>(PARTimg + off) = s;
                } else {
                  const float* sl = reinterpret_cast<const float*>(slots + xpar * NW * SLOT + f_it) + f_comp;
                  float s = sl[0];
#pragma unroll
                  for (int w = 1; w < NW; ++w) s += sl[2 * w * SLOT];
                  *reinterpret_cast<float*>(PARTimg + off) = s;
                }
              }
              xpar ^= 1;
            }
          }
        }
       }
        if constexpr (BATCH) {
          // ---- across the waves, both steps of this half-pass at once: the 2 x 3 (step, tensor) sets are dealt to the
          // waves; a thread adds up the float2 of the lane (its slot, its row).  The other half's sets are being
          // filled or added up by then; this half's are filled again two barriers from here.
          __syncthreads();
          if constexpr (STAGES)
#pragma unroll
          for (int rd = 0; rd < (2 * 3 + NSTG - 1) / NSTG; ++rd) {
            const int jj = rd * NSTG + swave;                 // (uniform)
            if (jj < 2 * 3) {
              const int ks = jj / 3, v = jj - 3 * ks;
              const int k = k0 + ks;
              if (t0 + k < p.T_total && ((bp.in_grid >> k) & 1u)) {
                const uint32_t off = f_off0 + (uint32_t)k * pstep + (k >= bp.kw ? pwrap_adj : 0u) + (uint32_t)((v * kN + 2 * half) * sizeof(float));
                const float2* sl = slots + (2 * half + ks) * NW * SLOT + v * 64 + lane;
                float2 sum = sl[0];
#pragma unroll
                for (int w = 1; w < NW; ++w) { sum.x += sl[w * SLOT].x; sum.y += sl[w * SLOT].y; }
                *reinterpret_cast<float2*>(PARTimg + off) = sum;
              }
            }
          }
        }
      }
    }
    if constexpr (!BATCH) __syncthreads();   // (BATCH: the barrier of the last half-pass ended the block)
    A = Aprev;
    bp = bpn;
    cell0 = celln;
    cur ^= 1;
    take0 = take0n; take1 = take1n;
  }
  };
  if constexpr (NH == 0) sweep(std::integral_constant<int, kAll>{});
  else if (helper) sweep(std::integral_constant<int, kStager>{});
  else sweep(std::integral_constant<int, kSweeper>{});

  // ---- sums over positions: reduce over the rows of the band (lanes of one channel slot)
  float red[2 * kN + 1];
#pragma unroll
  for (int n = 0; n < kN; ++n) { red[n] = accAT[n]; red[kN + n] = accAL[n]; }
  red[2 * kN] = accD;
#pragma unroll
  for (int k = 0; k < 2 * kN + 1; ++k) {
    float v = red[k];
#pragma unroll
    for (int off = kHB >> 1; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    red[k] = v;
  }
  if (ch_ok && r == 0) {
    const int64_t slot_e = (int64_t)b * p.pa_slots * p.E + e;
    float* pa = p.pA + slot_e * (2 * kN);
#pragma unroll
    for (int n = 0; n < 2 * kN; ++n) pa[n] = red[n];
    p.pD[slot_e] = red[2 * kN];
  }
}

// ------------------------------------------------------ backward, the states of a channel split over lanes
// The counterpart of m2d_fwd_split_kernel: lane = (state group g, row r), 4 states per lane, a wave
// per channel, 8 channels per workgroup.  With only 4 states a lane keeps the gates of all four
// steps of a block from the recomputation to the adjoint, and sweeps a block in one pass.  Sums over
// the states of a cell (for d_delta and d_x) are taken across the 4 lane groups by lane swaps; sums
// over channels (d_C, d_BT, d_BL) across the 8 waves through LDS, as in m2d_bwd_kernel, a float4 of
// four states per lane.  Memory formats are those of m2d_bwd_kernel.
template <typename T, bool STAGE_X, int MODE, int NWS = kSplitWaves>
__global__ __launch_bounds__((NWS + split_helpers<MODE, NWS, STAGE_X>()) * 64) void m2d_bwd_split_kernel(const ScanParams pin) {
  static_assert(MODE != kModeStacked, "stacked images are many: they never need the split");
  constexpr bool SLICED = MODE == kModeSliced;
  const ScanParams& p = pin;
  __builtin_assume(p.stacked == 0);
  __builtin_assume(p.rb == kRB);
  __builtin_assume(p.S >= kHB + kCK - 1);
  constexpr int NW = NWS, CW = NW;
  constexpr int NH = split_helpers<MODE, NWS, STAGE_X>();   // waves that only stage and add up the channel sums (then the first NW waves only sweep)
  constexpr int NSTG = NH ? NH : NW;               // waves that share the copies of a block
  static_assert(NH == 0 || NH >= 3, "three waves add up the channel sums");
  constexpr int SLOT = 3 * 64;           // float4s per wave in one exchange buffer
  using SG = Stage<T, 4, CW, true>;
  constexpr bool WIDEN = sizeof(T) == 2;
  extern __shared__ float4 smem[];
  float4* slots = smem;                                            // [2][wave][3][64], used alternately: one barrier per step
  char* lds = reinterpret_cast<char*>(slots + 2 * NW * SLOT);      // two staging buffers
  char* raw = lds + 2 * SG::kBytes;                                // [2][kRawBytes]
  const bool direct = WIDEN && p.bc_direct != 0;   // (uniform)
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  int lb = SLICED ? (int)blockIdx.x : logical_block(p.nwg);
  int m_lo = 0, m_hi = p.nblk;
  int my_band = 0;
  LinkT<NH ? NW * 64 : 0> link;
  if constexpr (SLICED) {   // the window of one band; the bands are launched from the last to the first
    const int per = p.B * p.bpb;
    const int kk = lb / per;
    lb -= kk * per;
    my_band = p.nbands - 1 - kk;
    m_lo = my_band * p.sl_nbb;
    m_hi = m_lo + p.sl_nbb;
    link.mine = p.prog + ((int64_t)my_band * per + lb) * kLinkStride;
    link.dep = my_band + 1 < p.nbands ? link.mine + per * kLinkStride : nullptr;
    link.err = p.link_err;
    link.rig(p, my_band);
  }
  const bool helper = NH && wave >= NW;      // (uniform) stages and adds up, never sweeps
  const bool stages = !NH || helper;
  const int swave = NH ? wave - NW : wave;   // the wave's turn among those that stage
  const int b = lb / p.bpb;
  const int eg = lb % p.bpb;
  const int e_wg0 = eg * CW;
  const int g = lane >> kHBShift, r = lane & (kHB - 1);
  const int rbands = row_bands(p, r);
  const int ch_loc = helper ? 0 : wave;
  const bool ch_ok = !helper && e_wg0 + ch_loc < p.E;   // (uniform)
  const int e = ch_ok ? e_wg0 + ch_loc : p.E - 1;
  for (int i = threadIdx.x; i < 2 * SG::kBytes / 16; i += (NW + NH) * 64) reinterpret_cast<float4*>(lds)[i] = make_float4(0.f, 0.f, 0.f, 0.f);
  // register w of the lane meets position 4g + w of a record: state perm(w) * 4 + g (fold order)
  int state_of[4];
  float a2t[4], a2l[4];
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    state_of[w] = (w == 1 ? 2 : (w == 2 ? 1 : w)) * 4 + g;
    a2t[w] = p.A2T[e * kN + state_of[w]];
    a2l[w] = p.A2L[e * kN + state_of[w]];
  }
  const float dsk = p.Df[e];
  settle_loads();

  const T* X = static_cast<const T*>(p.x);
  const T* DT = static_cast<const T*>(p.dT);
  const T* DL = static_cast<const T*>(p.dL);
  const T* DY = static_cast<const T*>(p.dy);
  const int64_t img_cell0 = (int64_t)b * p.Hs * p.W;
  const int64_t img_bytes = img_cell0 * p.E * (int64_t)sizeof(T);
  const char* Ximg = reinterpret_cast<const char*>(X) + img_bytes;
  const char* DTimg = reinterpret_cast<const char*>(DT) + img_bytes;
  const char* DLimg = reinterpret_cast<const char*>(DL) + img_bytes;
  const char* DYimg = reinterpret_cast<const char*>(DY) + img_bytes;
  // the three per-cell results are stored by three of the four lane groups: group 0 d_deltaT, 2 d_deltaL, 1 d_x
  char* OUTimg = (g == 0 ? static_cast<char*>(p.ddT) : (g == 2 ? static_cast<char*>(p.ddL) : static_cast<char*>(p.dx))) + img_bytes;
  char* BOTimg = reinterpret_cast<char*>(p.bot + (int64_t)b * p.W * p.E * kN);   // + band * bot_stride
  char* PARTimg = reinterpret_cast<char*>(p.part + ((int64_t)eg * p.Ptot + img_cell0) * (3 * kN));

  float accAT[4], accAL[4], accD = 0.f, muT[4], muL[4];
#pragma unroll
  for (int w = 0; w < 4; ++w) { accAT[w] = 0.f; accAL[w] = 0.f; muT[w] = 0.f; muL[w] = 0.f; }
  // the lane's group of (B_T, B_L, C): a grid row reads those of its cell; the upper ghost (lane 0) the row
  // above as its B_T; the lower ghost (lane 15) the row of mu_T below as its C (see m2d_bwd_kernel)
  const uint32_t rec_off = (r == 0 ? SG::top_off(ch_loc) : (r == kHB - 1 ? SG::bot_off(ch_loc) - SG::kCOff : r * 16)) + g * SG::kPlane;
  const uint32_t const_off = SG::kConstPlane * SG::kPlane + r * 16;
  const uint32_t xd_off = SG::kXOff + SG::x_off(r, ch_loc + (CW < SG::kElem ? e_wg0 & (SG::kElem - 1) : 0));   // (4 channels of a 16-bit tensor: their half of the chunk)
  constexpr uint32_t kXK = SG::kXStepBytes;
  // channel sums: the first 6 waves add up; wave 2v + c takes components 2c, 2c+1 of every lane's float4 of
  // tensor v.  They are kept per cell as [C, B_T, B_L][16] in the natural order of the states.
  // (workgroups of 4 waves: the first 3 add up, a whole float4 each)
  // (with waves that only stage: the first 3 of those, a whole float4 each)
  constexpr bool QUADS = NH > 0 || NW < 6;
  const bool f_on = NH ? (helper && swave < 3) : wave < (QUADS ? 3 : 6);
  const int f_v = QUADS ? swave : wave >> 1, f_c = QUADS ? 0 : wave & 1;
  const uint32_t f_sub0 = (uint32_t)(f_v * kN + (f_c ? 1 : 0) * 4 + g) * (uint32_t)sizeof(float);   // component 2c: state perm(2c) * 4 + g, perm = (0, 2, 1, 3)
  const uint32_t f_sub1 = (uint32_t)(f_v * kN + (f_c ? 3 : 2) * 4 + g) * (uint32_t)sizeof(float);   // component 2c + 1
  const float g1 = r == 0 ? 1.f : 0.f;
  const float gb1 = r == kHB - 1 ? 1.f : 0.f;
  const uint32_t estep = (uint32_t)(p.flip ? -p.E : p.E) * (uint32_t)sizeof(T);
  const uint32_t wrap_adj = (uint32_t)(p.rb * p.W - p.S) * estep;
  const uint32_t pstep = (uint32_t)(p.flip ? -1 : 1) * (uint32_t)(3 * kN * sizeof(float));
  const uint32_t pwrap_adj = (uint32_t)(p.rb * p.W - p.S) * pstep;

  BlockPos bp;
  uint32_t cell_off0 = 0, f_off0 = 0;
  typename Snap<T>::quad cknext = Snap<T>::zero();
  auto load_ckpt = [&](int mm, bool take) {   // take: the forward kept the lane's state before block mm
    cknext = Snap<T>::zero();
    if (mm != 0 && take) {
      int ln = lane;
      asm volatile("" : "+v"(ln));   // the lane's place is worked out here, not carried in a register across the block (the kernel has none to spare)
      cknext = *(snapshot_at<T>(p, b, mm, e, p.nblk) + snap_lane(ln & (kHB - 1)) + snap_quad(ln >> kHBShift));
    }   // (this kernel: a snapshot for every block)
  };
  auto pos_before = [&](Pos Q) {
    Q.col -= kCK;
    if (Q.col < 0) { Q.col += p.S; Q.bnd -= 1; }
    return Q;
  };

  Pos A = pos_of(p, (m_hi - 1) * kCK - (kHB - 1));
  __syncthreads();   // the zeros are in place before the first copies land on them
  bp = block_pos(p, A, r, rbands);
  int cell0 = cell_of(p, bp.bnd0, r, bp.col0);
  bool ck_take = snapshot_lane(p, Pos{bp.bnd0, bp.col0}, r, ch_ok);
  load_ckpt(m_hi - 1, ck_take);
  if constexpr (SLICED) { if (stages) link.wait_for(link_need_bwd(p.sl_nbb - 1, p.sl_nbb)); }
  auto raw_copy_for = [&](Pos A2, char* dst, bool live) {
    if (!stages) return;   // (uniform)
    const BlockPos q2 = block_pos(p, A2, r, rbands);
    bc_raw_copy<NSTG>(p, pin.bcd, dst, b, q2, cell_of(p, q2.bnd0, r, q2.col0), swave, lane, live);
  };
  int rp = 0;
  if (direct) {
    if (stages) bc_raw_copy<NSTG>(p, pin.bcd, raw, b, bp, cell0, swave, lane, true);
    raw_copy_for(pos_before(A), raw + kRawBytes, m_hi - 2 >= m_lo);
    if (stages) stage_block<T, 4, CW, true, STAGE_X, NSTG, true>(p, lds, b, A, bp, cell0, e_wg0, swave, lane, X, DT, DL, DY);
    staging_fence();
    if (stages) bc_widen<SG, NSTG>(raw, lds, swave, lane);
  } else {
    if (stages) stage_block<T, 4, CW, true, STAGE_X, NSTG>(p, lds, b, A, bp, cell0, e_wg0, swave, lane, X, DT, DL, DY);
  }
  staging_fence();
  int cur = 0;
  int xpar = 0;

  // The sweep over the blocks of the window, as a wave of the given role runs it (see m2d_fwd_split_kernel); the
  // waves that stage also add up the channel sums of every step.
  auto sweep = [&](auto role) {
  constexpr int ROLE = decltype(role)::value;
  constexpr bool STAGES = ROLE != kSweeper, SWEEPS = ROLE != kStager;
  for (int m = m_hi - 1; m >= m_lo; --m) {
    const int t0 = m * kCK;
    const char* bufc = lds + cur * SG::kBytes;
    float hb[kCK + 1][4], gT[kCK][4], gL[kCK][4];
    if constexpr (SWEEPS) { const float4 v = Snap<T>::widen(cknext); hb[0][0] = v.x; hb[0][1] = v.y; hb[0][2] = v.z; hb[0][3] = v.w; }
    const Pos Aprev = pos_before(A);
    const BlockPos bpn = block_pos(p, Aprev, r, rbands);
    const int celln = cell_of(p, bpn.bnd0, r, bpn.col0);
    if constexpr (SWEEPS) ck_take = snapshot_lane(p, Pos{bpn.bnd0, bpn.col0}, r, ch_ok);
    if constexpr (STAGES) { if (direct) raw_copy_for(pos_before(Aprev), raw + rp * kRawBytes, m - 2 >= m_lo); }
    if (STAGES && m > m_lo) {
      if constexpr (SLICED) link.wait_for(link_need_bwd(m - 1 - m_lo, p.sl_nbb));
      if (direct) {
        stage_block<T, 4, CW, true, STAGE_X, NSTG, true>(p, lds + (cur ^ 1) * SG::kBytes, b, Aprev, bpn, celln, e_wg0, swave, lane, X, DT, DL, DY);
        bc_widen<SG, NSTG>(raw + (rp ^ 1) * kRawBytes, lds + (cur ^ 1) * SG::kBytes, swave, lane);
      } else {
        stage_block<T, 4, CW, true, STAGE_X, NSTG>(p, lds + (cur ^ 1) * SG::kBytes, b, Aprev, bpn, celln, e_wg0, swave, lane, X, DT, DL, DY);
      }
    }
    rp ^= 1;
    if constexpr (SWEEPS) cell_off0 = (uint32_t)(cell0 * p.E + e) * (uint32_t)sizeof(T);
    if constexpr (STAGES) f_off0 = (uint32_t)cell0 * (uint32_t)(3 * kN * sizeof(float));

    // ---- recompute the states of the block, keeping the gates
    if constexpr (SWEEPS)
#pragma unroll
    for (int k = 0; k < kCK; ++k) {
      if (t0 + k < p.T_total) {
        const float4 kk = *reinterpret_cast<const float4*>(bufc + const_off + k * SG::kKStr);
        const float offT = kk.x, offL = kk.y, cT = kk.z, cL = kk.w;
        float xv = 0.f, dtv = 0.f, dlv = 0.f;
        if constexpr (STAGE_X) {
          const T* xr = reinterpret_cast<const T*>(bufc + xd_off + k * kXK);
          xv = IO<T>::ld(xr); dtv = IO<T>::ld(xr + SG::kXTauBytes / sizeof(T)); dlv = IO<T>::ld(xr + 2 * SG::kXTauBytes / sizeof(T));
        } else if (ch_ok && ((bp.in_grid >> k) & 1u)) {
          const uint32_t off = cell_off0 + (uint32_t)k * estep + (k >= bp.kw ? wrap_adj : 0u);
          xv = IO<T>::ld(reinterpret_cast<const T*>(Ximg + off));
          dtv = IO<T>::ld(reinterpret_cast<const T*>(DTimg + off));
          dlv = IO<T>::ld(reinterpret_cast<const T*>(DLimg + off));
        }
        const char* rec = bufc + (rec_off + k * SG::kKStr);
        const float4 b4 = *reinterpret_cast<const float4*>(rec);
        const float4 l4 = *reinterpret_cast<const float4*>(rec + SG::kBLOff);
        const float bq[4] = {b4.x, b4.y, b4.z, b4.w}, lq[4] = {l4.x, l4.y, l4.z, l4.w};
        const float sT = __builtin_fmaf(cT * dtv, xv, g1);
        const float sL = cL * dlv * xv;
#pragma unroll
        for (int w = 0; w < 4; ++w) gT[k][w] = fexp2(__builtin_fmaf(dtv, a2t[w], offT));
        pin4(gT[k]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int w = 0; w < 4; ++w) gL[k][w] = fexp2(__builtin_fmaf(dlv, a2l[w], offL));
        pin4(gL[k]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          float u = sL * lq[w];
          u = __builtin_fmaf(sT, bq[w], u);
          u = fma_row_below(gT[k][w], hb[k][w], u);
          hb[k + 1][w] = __builtin_fmaf(gL[k][w], hb[k][w], u);
        }
      } else {
#pragma unroll
        for (int w = 0; w < 4; ++w) { gT[k][w] = 0.f; gL[k][w] = 0.f; hb[k + 1][w] = 0.f; }
      }
    }
    // ---- adjoint over the block, last step first
#pragma unroll
    for (int k = kCK - 1; k >= 0; --k) {
      if (k == 0) staging_landed();   // before the last stores of the block
      if constexpr (SWEEPS) { if (k == (kCK > 1 ? 1 : 0) && m > m_lo) load_ckpt(m - 1, ck_take); }
      if (t0 + k < p.T_total) {
       if constexpr (SWEEPS) {
        const float4 kk = *reinterpret_cast<const float4*>(bufc + const_off + k * SG::kKStr);
        const float cT = kk.z, cL = kk.w;
        const bool inr = ch_ok && ((bp.in_grid >> k) & 1u);
        const uint32_t goff = cell_off0 + (uint32_t)k * estep + (k >= bp.kw ? wrap_adj : 0u);
        float xv = 0.f, dtv = 0.f, dlv = 0.f, dyv = 0.f;
        if constexpr (STAGE_X) {
          const T* xr = reinterpret_cast<const T*>(bufc + xd_off + k * kXK);
          xv = IO<T>::ld(xr); dtv = IO<T>::ld(xr + SG::kXTauBytes / sizeof(T)); dlv = IO<T>::ld(xr + 2 * SG::kXTauBytes / sizeof(T));
          dyv = IO<T>::ld(xr + 3 * SG::kXTauBytes / sizeof(T));
        } else if (inr) {
          xv = IO<T>::ld(reinterpret_cast<const T*>(Ximg + goff));
          dtv = IO<T>::ld(reinterpret_cast<const T*>(DTimg + goff));
          dlv = IO<T>::ld(reinterpret_cast<const T*>(DLimg + goff));
          dyv = IO<T>::ld(reinterpret_cast<const T*>(DYimg + goff));
        }
        const char* rec = bufc + (rec_off + k * SG::kKStr);
        const float4 b4 = *reinterpret_cast<const float4*>(rec);
        const float4 l4 = *reinterpret_cast<const float4*>(rec + SG::kBLOff);
        const float4 c4 = *reinterpret_cast<const float4*>(rec + SG::kCOff);
        const float bq[4] = {b4.x, b4.y, b4.z, b4.w}, lq[4] = {l4.x, l4.y, l4.z, l4.w}, cq[4] = {c4.x, c4.y, c4.z, c4.w};
        const float qT = cT * dtv * xv, qL = cL * dlv * xv;   // zero on lanes that are not grid cells
        const float dyl = dyv + gb1;
        float sT = 0.f, sL = 0.f, zT = 0.f, zL = 0.f;
        float vC[4], vBT[4], vBL[4];
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          const float lam = __builtin_fmaf(dyl, cq[w], add_row_above(muL[w], muT[w]));
          const float mT = gT[k][w] * lam, mL = gL[k][w] * lam;
          muT[w] = mT;
          muL[w] = mL;
          const float ZT = mul_row_below(mT, hb[k][w]), ZL = mL * hb[k][w];
          accAT[w] = __builtin_fmaf(ZT, dtv, accAT[w]);
          accAL[w] = __builtin_fmaf(ZL, dlv, accAL[w]);
          zT = __builtin_fmaf(ZT, a2t[w], zT);
          zL = __builtin_fmaf(ZL, a2l[w], zL);
          sT = __builtin_fmaf(lam, bq[w], sT);
          sL = __builtin_fmaf(lam, lq[w], sL);
          vBT[w] = qT * lam;
          vBL[w] = qL * lam;
          vC[w] = dyv * hb[k + 1][w];
        }
        float4* sw = slots + (xpar * NW + wave) * SLOT + lane;
        sw[0] = make_float4(vC[0], vC[1], vC[2], vC[3]);
        sw[64] = make_float4(vBT[0], vBT[1], vBT[2], vBT[3]);
        sw[128] = make_float4(vBL[0], vBL[1], vBL[2], vBL[3]);
        if (p.nbands > 1) {   // first row of a band: the lower ghost of the band above will replay its muT
          const bool wk = k >= bp.kw;
          if (inr && r == 1 && (wk ? bp.bnd0 + 1 : bp.bnd0) >= 1) {
            const int ck = wk ? bp.col0 + k - p.S : bp.col0 + k;
            float4* bb = reinterpret_cast<float4*>(BOTimg + (wk ? bp.bnd0 + 1 : bp.bnd0) * p.bot_stride * (int64_t)sizeof(float) +
                                                   (uint32_t)(ck * p.E + e) * (uint32_t)(kN * sizeof(float))) + g;
            const float4 row = make_float4(muT[0], muT[1], muT[2], muT[3]);
            if constexpr (SLICED) store_row_device_scope(bb, row); else *bb = row;
          }
        }
        // the lane's share (its 4 states) of d_deltaT, d_deltaL and d_x of the cell; summed over the 4
        // groups, the totals arrive in the lanes of group 0, 2 and 1
        const float pT = __builtin_fmaf(cT * xv, sT, kLn2 * zT);
        const float pL = __builtin_fmaf(cL * xv, sL, kLn2 * zL);
        const float pX = __builtin_fmaf(cT * dtv, sT, cL * dlv * sL);
        float tot = fold16(fold32(pT, pL), fold32(pX, 0.f));
        accD = __builtin_fmaf(dyv, xv, accD);
        if (p.dpre && (g & 1) == 0) tot *= softplus_slope<T>(g == 0 ? dtv : dlv);   // gradients with respect to what the softplus was applied to
        if (g == 1) tot = __builtin_fmaf(dyv, dsk, tot);
        if (inr && g != 3) IO<T>::st(reinterpret_cast<T*>(OUTimg + goff), tot);
       }
        // ---- across the waves of the workgroup
        __syncthreads();
        if (STAGES && f_on && ((bp.in_grid >> k) & 1u)) {
          const uint32_t off = f_off0 + (uint32_t)k * pstep + (k >= bp.kw ? pwrap_adj : 0u);
          if constexpr (QUADS) {
            const float4* sl = slots + xpar * NW * SLOT + f_v * 64 + lane;
            float4 sum = sl[0];
#pragma unroll
            for (int w = 1; w < NW; ++w) { const float4 o = sl[w * SLOT]; sum.x += o.x; sum.y += o.y; sum.z += o.z; sum.w += o.w; }
            // component j holds state perm(j) * 4 + g, perm = (0, 2, 1, 3)
            float* dst = reinterpret_cast<float*>(PARTimg + off + (uint32_t)(f_v * kN + g) * (uint32_t)sizeof(float));
            dst[0] = sum.x; dst[8] = sum.y; dst[4] = sum.z; dst[12] = sum.w;
          } else {
            const float2* sl = reinterpret_cast<const float2*>(slots + xpar * NW * SLOT + f_v * 64 + lane) + f_c;
            float2 sum = sl[0];
#pragma unroll
            for (int w = 1; w < NW; ++w) { sum.x += sl[2 * w * SLOT].x; sum.y += sl[2 * w * SLOT].y; }
            *reinterpret_cast<float*>(PARTimg + off + f_sub0) = sum.x;
            *reinterpret_cast<float*>(PARTimg + off + f_sub1) = sum.y;
          }
        }
        xpar ^= 1;
      }
    }
    __syncthreads();
    if constexpr (SLICED && STAGES) link.publish((uint32_t)(m_hi - m));   // (this block counts: see m2d_bwd_kernel)
    A = Aprev;
    bp = bpn;
    cell0 = celln;
    cur ^= 1;
  }
  };
  if constexpr (NH == 0) sweep(std::integral_constant<int, kAll>{});
  else if (helper) sweep(std::integral_constant<int, kStager>{});
  else sweep(std::integral_constant<int, kSweeper>{});
  bool broken = false;
  if constexpr (SLICED) {
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    link.publish((uint32_t)p.sl_nbb);
    broken = link.broken() || link_poll(p.link_err) != 0u;   // (also a workgroup of the forward sweep that rebuilt the snapshots for this launch)
    if constexpr (NH > 0) {   // only the waves that wait know of a wait given up: they tell the others (the staging buffers are free now)
      if ((int)threadIdx.x == link.pub) *reinterpret_cast<volatile uint32_t*>(lds) = link.broken() ? 1u : 0u;
      __syncthreads();
      broken = broken || *reinterpret_cast<volatile uint32_t*>(lds) != 0u;
    }
    if (broken) poison_band<T>(p, my_band, b, e_wg0, CW, p.dx, p.ddT, p.ddL);
  }

  // ---- sums over positions: reduce over the rows of the band (the 16 lanes of a group)
  float red[9];
#pragma unroll
  for (int w = 0; w < 4; ++w) { red[w] = accAT[w]; red[4 + w] = accAL[w]; }
  red[8] = broken ? __builtin_nanf("") : accD;
  if (broken) { red[0] = __builtin_nanf(""); red[4] = __builtin_nanf(""); }   // (d_AT, d_AL, d_D of the channel say so too)
#pragma unroll
  for (int k = 0; k < 9; ++k) {
    float v = red[k];
#pragma unroll
    for (int off = kHB >> 1; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    red[k] = v;
  }
  if (ch_ok && r == 0) {
    const int64_t slot_e = ((int64_t)b * p.pa_slots + (SLICED ? my_band : 0)) * p.E + e;
    float* pa = p.pA + slot_e * (2 * kN);
#pragma unroll
    for (int w = 0; w < 4; ++w) { pa[state_of[w]] = red[w]; pa[kN + state_of[w]] = red[4 + w]; }
    if (g == 0) p.pD[slot_e] = red[8];
  }
}

// -------------------------------------------------------------------------- small helper kernels
// the value a tensor of type T would hold
__device__ __forceinline__ float as_stored(float v, const float*) { return v; }
__device__ __forceinline__ float as_stored(float v, const bf16_t*) { return bf16_bits_to_f32(f32_to_bf16_bits(v)); }

// RAW: the parameters as the module holds them (fp32 A_log, fp32 D): A = -exp(A_log), and both
// are rounded to T, which is what the reference's casts to x.dtype do (wavefront_cuda.py:72-73,
// 90-91, 332).
template <typename T, bool RAW>
__global__ void m2d_prep_kernel(const void* ATv, const void* ALv, const void* Dv, float* zeros, float* A2T, float* A2L, float* Df, int E,
                                uint32_t* link_words, int n_link_words) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx < kZeroFloats) zeros[idx] = 0.f;
  // linked sweep: error word and progress counts start at zero
  for (int i = idx; i < n_link_words; i += gridDim.x * blockDim.x) link_words[i] = 0u;
  if constexpr (RAW) {
    const float *AT = static_cast<const float*>(ATv), *AL = static_cast<const float*>(ALv), *D = static_cast<const float*>(Dv);
    if (idx < E * kN) {
      A2T[idx] = as_stored(-expf(AT[idx]), static_cast<const T*>(nullptr)) * kLog2e;
      A2L[idx] = as_stored(-expf(AL[idx]), static_cast<const T*>(nullptr)) * kLog2e;
    }
    if (idx < E) Df[idx] = as_stored(D[idx], static_cast<const T*>(nullptr));
  } else {
    const T *AT = static_cast<const T*>(ATv), *AL = static_cast<const T*>(ALv), *D = static_cast<const T*>(Dv);
    if (idx < E * kN) {
      A2T[idx] = IO<T>::ld(AT + idx) * kLog2e;
      A2L[idx] = IO<T>::ld(AL + idx) * kLog2e;
    }
    if (idx < E) Df[idx] = IO<T>::ld(D + idx);
  }
}

// B_T, B_L, C -> one fp32 record of 48 values per cell (three runs of 16, each in fold order,
// see spos), so the scan kernels read their operands a float4 per state group.
template <typename T>
__global__ void m2d_pack_bc_kernel(const T* BT, const T* BL, const T* C, float* out, int64_t P) {
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;   // one thread per (cell, tensor)
  if (gid >= P * 3) return;
  const int64_t cell = gid / 3;
  const int tsr = (int)(gid % 3);
  const T* src = (tsr == 0 ? BT : (tsr == 1 ? BL : C)) + cell * kN;
  float v[kN];
  if constexpr (sizeof(T) == 2) {
    const uint4 t0 = reinterpret_cast<const uint4*>(src)[0], t1 = reinterpret_cast<const uint4*>(src)[1];
    const uint32_t wds[8] = {t0.x, t0.y, t0.z, t0.w, t1.x, t1.y, t1.z, t1.w};
#pragma unroll
    for (int k = 0; k < 8; ++k) { v[2 * k] = __uint_as_float(wds[k] << 16); v[2 * k + 1] = __uint_as_float(wds[k] & 0xffff0000u); }
  } else {
    ld16f(reinterpret_cast<const float*>(src), v);
  }
  float4* dst = reinterpret_cast<float4*>(out + cell * 48 + tsr * kN);
#pragma unroll
  for (int q = 0; q < 4; ++q)
    dst[q] = make_float4(v[sinv<true>(4 * q)], v[sinv<true>(4 * q + 1)], v[sinv<true>(4 * q + 2)], v[sinv<true>(4 * q + 3)]);
}

// d_C, d_BT, d_BL: add the per-workgroup channel sums in workgroup order and round to T.
// d_AT, d_AL, d_D: add the per-image partials in image order.
// RAW: d_AT, d_AL, d_D are fp32 and refer to the parameters as the module holds them:
// A = -exp(A_log), so d_A_log = d_A * A (A is at hand as A2 / log2 e).
template <typename T, bool RAW>
__global__ void m2d_finalize_kernel(const ScanParams p, T* dC, T* dBT, T* dBL, void* dATv, void* dALv, void* dDv, int parts_stay) {
  const int64_t P = p.Ptot;
  const int64_t nquad = parts_stay ? 0 : 3 * P * (kN / 4);   // (parts_stay: the reader of d_C, d_BT, d_BL adds up the per-workgroup sums itself)
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid < nquad) {
    // per-workgroup sums are laid out [channel group][cell][C, B_T, B_L][16]: consecutive threads
    // read consecutive float4s
    const int64_t cell = gid / 12;
    const int rem = (int)(gid - cell * 12), v = rem >> 2, q = rem & 3;
    const float* src = p.part + cell * (3 * kN) + rem * 4;
    float4 s = *reinterpret_cast<const float4*>(src);
    for (int egi = 1; egi < p.bpb; ++egi) {
      const float4 o = *reinterpret_cast<const float4*>(src + (int64_t)egi * P * 3 * kN);
      s.x += o.x; s.y += o.y; s.z += o.z; s.w += o.w;
    }
    T* out = v == 0 ? dC : (v == 1 ? dBT : dBL);
    IO<T>::st4(out + cell * kN + q * 4, s);
  }
  // d_AT, d_AL, d_D: the blocks after the last block of quads add up the per-image partials, 16
  // lanes to a sum (lane l takes images l, l+16, ...; the 16 partial sums are folded in a fixed
  // order), so that the loads of one sum are in flight together.
  const int64_t tail = gid - (nquad + blockDim.x - 1) / blockDim.x * blockDim.x;
  if (tail >= 0) {
    const int64_t out = tail >> 4;
    const int l = (int)(tail & 15);
    const int nA = p.B * p.pa_slots;
    const int64_t n_at = (int64_t)p.E * 2 * kN;
    float s = 0.f;
    if (out < n_at) {
      const int e = (int)(out / (2 * kN)), w = (int)(out % (2 * kN));
      for (int g = l; g < nA; g += 16) s += p.pA[((int64_t)g * p.E + e) * (2 * kN) + w];
    } else if (out < n_at + p.E) {
      for (int g = l; g < nA; g += 16) s += p.pD[(int64_t)g * p.E + (out - n_at)];
    }
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
    if (l == 0) {
      if (out < n_at) {
        const int e = (int)(out / (2 * kN)), w = (int)(out % (2 * kN));
        if constexpr (RAW) {
          if (w < kN) static_cast<float*>(dATv)[e * kN + w] = s * p.A2T[e * kN + w] * kLn2;
          else static_cast<float*>(dALv)[e * kN + (w - kN)] = s * p.A2L[e * kN + (w - kN)] * kLn2;
        } else {
          if (w < kN) IO<T>::st(static_cast<T*>(dATv) + e * kN + w, s); else IO<T>::st(static_cast<T*>(dALv) + e * kN + (w - kN), s);
        }
      } else if (out < n_at + p.E) {
        if constexpr (RAW) static_cast<float*>(dDv)[out - n_at] = s;
        else IO<T>::st(static_cast<T*>(dDv) + (out - n_at), s);
      }
    }
  }
}


// ------------------------------------------------------------------ instruction-rate probe
// What the vector ALUs of this device issue per second, measured (m2d_valu_rate_probe): the scan kernels are
// bound by instruction issue, and the ceiling they are priced against should not be a nominal clock times a lane
// count.  Every lane runs kProbeIters x 16 operations of one kind on values that stay in registers:
//   independent: 16 chains per lane (what a kernel with enough parallel work in a lane sees),
//   dependent:   one chain per lane (every operation waits for the one before),
// for v_fma_f32 and for v_exp_f32, and the forward scan's own mix per (cell, channel, state): two gate
// exponents with their multiply-adds and the five multiply-adds of the state and output update.
constexpr int kProbeIters = 4096;
template <int KIND>
__global__ __launch_bounds__(256) void m2d_rate_probe_kernel(float* out, float a, float b) {
  float r[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) r[i] = -(threadIdx.x * 0.001f + i) * 0.01f;
  if constexpr (KIND == M2D_RATE_FMA) {
    for (int it = 0; it < kProbeIters; ++it)
#pragma unroll
      for (int i = 0; i < 16; ++i) r[i] = __builtin_fmaf(r[i], a, b);
  } else if constexpr (KIND == M2D_RATE_FMA_DEPENDENT) {
    for (int it = 0; it < kProbeIters; ++it)
#pragma unroll
      for (int i = 0; i < 16; ++i) r[0] = __builtin_fmaf(r[0], a, b);
  } else if constexpr (KIND == M2D_RATE_EXP) {
    for (int it = 0; it < kProbeIters; ++it)
#pragma unroll
      for (int i = 0; i < 16; ++i) r[i] = fexp2(r[i]);
  } else if constexpr (KIND == M2D_RATE_EXP_DEPENDENT) {
    for (int it = 0; it < kProbeIters; ++it)
#pragma unroll
      for (int i = 0; i < 16; ++i) r[0] = fexp2(r[0]);
  } else {   // M2D_RATE_SCAN_FWD_UNIT: r are 16 states; one iteration is one step of a cell and channel
    float acc = 0.f, d = a, sT = b, sL = a * b;
    for (int it = 0; it < kProbeIters; ++it) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float gT = fexp2(__builtin_fmaf(d, -0.01f * (i + 1), -1.f));
        const float gL = fexp2(__builtin_fmaf(sT, -0.02f * (i + 1), -1.f));
        float u = sL * (0.5f + i);
        u = __builtin_fmaf(sT, 0.25f * i, u);
        u = __builtin_fmaf(gT, r[(i + 1) & 15], u);
        r[i] = __builtin_fmaf(gL, r[i], u);
        acc = __builtin_fmaf(r[i], d, acc);
      }
      // (the step's operands change from step to step, as a cell's do: nothing of a unit can leave the loop)
      d = __builtin_fmaf(acc, 1e-30f, d);
      sT = __builtin_fmaf(acc, 2e-30f, sT);
      sL = __builtin_fmaf(acc, 3e-30f, sL);
    }
    r[0] += acc;
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) s += r[i];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

// ------------------------------------------------------------------------------------ host side
// Optional timing of the main kernel of each pass (off by default; see m2d_profile_enable).
bool g_profile = false;
hipEvent_t g_ev[2][2] = {{nullptr, nullptr}, {nullptr, nullptr}};

inline size_t align_up(size_t v, size_t a = 256) { return (v + a - 1) / a * a; }

// Dynamic LDS of a workgroup: the forward's two staging buffers, the backward's exchange buffers, its
// copy of A and two staging buffers.  A compute unit has 160 KB.
constexpr size_t kLdsPerWorkgroup = 160 * 1024;
template <typename T, int EC, int NW = kFwdWaves>
constexpr size_t fwd_lds_bytes() {
  return 2 * (size_t)Stage<T, 3, NW * 4 * EC, false>::kBytes + (sizeof(T) == 2 ? 2 * kRawBytes : 0) + 2 * (size_t)YTile<T, EC, NW>::kBytes + YTile<T, EC, NW>::kTableBytes;
}
template <typename T, int NW = kBwdWaves>
constexpr size_t bwd_lds_bytes() {
  return sizeof(float2) * bwd_exchange_sets<T, NW>() * NW * 3 * 64 + sizeof(float) * NW * 4 * 2 * kN + 256 +
         2 * (size_t)Stage<T, 4, NW * 4, true>::kBytes + (sizeof(T) == 2 ? 2 * kRawBytes : 0);
}
static_assert(fwd_lds_bytes<float, 1>() <= kLdsPerWorkgroup && fwd_lds_bytes<bf16_t, 1>() <= kLdsPerWorkgroup, "forward staging must fit the LDS");
static_assert(bwd_lds_bytes<float>() <= kLdsPerWorkgroup && bwd_lds_bytes<bf16_t>() <= kLdsPerWorkgroup, "backward staging must fit the LDS");

struct Geometry {
  int HB, hb_shift, CS, nbands, nblk;
  int S, T_total, rows_last;         // stream stride, total steps, rows of the last band
  int rb;                            // grid rows per band
  int fwd_ec, fwd_nw, fwd_wpb, fwd_bpb;   // forward: channels per lane, waves per workgroup, waves and workgroups per image
  int bwd_nw, bwd_wpb, bwd_bpb;      // backward: waves per workgroup, waves and workgroups (channel groups) per image
  bool fwd_split, bwd_split;         // the states of a channel split over the lanes (a wave per channel: m2d_fwd_split_kernel, m2d_bwd_split_kernel)
  bool stage_x;                      // x, delta, dy rows are whole 16-byte chunks: stage them through LDS
  bool sliced;                       // linked sweep: bands on workgroups of their own, handing boundary rows to each other inside one launch
  bool stacked;                      // images of one band stacked into tall images of independent bands
  int ips, vB, vH;                   // images per stack; number and height of what the kernels sweep
  int nbb;                           // linked sweep: blocks per band
  size_t link_bytes;                 // linked sweep: error word and the two arrays of progress counts (forward, backward)
  int ck_shift, ck_pb, ck_nblk;      // checkpoint interval: log2 of the blocks per kept snapshot; kept snapshots per band (linked sweep) and per image
  bool ck_half;                      // a snapshot every 2 steps: m2d_fwd_kernel<..., HALF> and m2d_bwd2_kernel
  bool snap32;                       // bf16 tensors with fp32 snapshots (M2D_FLAG_FP32_SNAPSHOTS)
  size_t ring_bytes;                 // backward with a longer interval: the replayed snapshots of every workgroup
  bool packed_bc;
  size_t prep_bytes, bc_bytes, ckpt_diag_bytes, top_bytes, bot_bytes, part_bytes, pa_bytes, pd_bytes;
};

int check_desc(const m2d_desc* d) {
  if (!d) return M2D_ERR_NULL_POINTER;
  if (d->B < 1 || d->E < 1 || d->N < 1 || d->H < 2 || d->W < 2) return M2D_ERR_BAD_SHAPE;
  if (d->N != kN) return M2D_ERR_UNSUPPORTED;
  if (d->dtype != M2D_F32 && d->dtype != M2D_BF16) return M2D_ERR_UNSUPPORTED;
  if ((d->ckpt_interval != 0 && d->ckpt_interval != 2 && d->ckpt_interval != 4 && d->ckpt_interval != 8 && d->ckpt_interval != 16) || (d->flags & ~(M2D_FLAG_FLIP | M2D_FLAG_RAW_PARAMS | M2D_FLAG_PACKED_BC | M2D_FLAG_DPRE | M2D_FLAG_SPLIT_STATES | M2D_FLAG_WHOLE_STATES | M2D_FLAG_TEST_DEAD_LINK | M2D_FLAG_SUM_PARTS | M2D_FLAG_FP32_SNAPSHOTS))) return M2D_ERR_UNSUPPORTED;
  if ((d->flags & M2D_FLAG_FP32_SNAPSHOTS) && d->dtype == M2D_BF16 && (d->ckpt_interval == 2 || d->ckpt_interval == 8 || d->ckpt_interval == 16)) return M2D_ERR_UNSUPPORTED;   // (fp32 snapshots: every 4 steps)
  if ((d->flags & M2D_FLAG_SPLIT_STATES) && (d->flags & M2D_FLAG_WHOLE_STATES)) return M2D_ERR_UNSUPPORTED;
  if ((int64_t)d->B * d->H * d->W >= ((int64_t)1 << 40)) return M2D_ERR_BAD_SHAPE;
  // one image is addressed with 32-bit byte offsets from its base (fp32: 4 bytes per element;
  // the widest per-cell record, the channel sums, is 192 bytes)
  if ((int64_t)d->H * d->W * d->E >= ((int64_t)1 << 30) || (int64_t)d->H * d->W >= ((int64_t)1 << 24)) return M2D_ERR_UNSUPPORTED;
  return M2D_OK;
}

// Compute units of the current device, asked once per process (256 on MI355X, which is also what
// a host without a GPU plans with: sizes queried there are the sizes of an MI355X).
int device_cus() {
  static const int n = [] {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess || prop.multiProcessorCount < 1) {
      (void)hipGetLastError();   // no device: not an error of a later call
      return 256;
    }
    return prop.multiProcessorCount;
  }();
  return n;
}

Geometry make_geometry(const m2d_desc* d) {
  Geometry g;
  const int64_t ncu = device_cus();
  g.HB = kHB;
  g.hb_shift = kHBShift;
  g.CS = 64 / g.HB;
  const int groups = (d->E + kBwdWaves * g.CS - 1) / (kBwdWaves * g.CS);   // workgroups per image
  // Grids of a single band (14x14, 7x7, 10x10 ...): a sweep spends as many steps filling and
  // draining the 16-lane pipeline as working.  `ips` consecutive images of the batch are then
  // stacked into one tall image whose bands do not depend on each other and swept back to back with
  // stride S = W; a band holds as many whole images as fit the 16 lanes (two of 7 or 8 rows, one of
  // 10 or 16, five of 3: no row above or below a band is needed, so the two outer lanes are rows
  // too), so no image straddles two bands.  ips is chosen for the fewest steps over all rounds of
  // workgroups (one workgroup per CU at a time).
  g.stacked = false; g.ips = 1; g.vB = d->B; g.vH = d->H;
  g.rb = kRB;
  const int rb_stacked = d->H <= kHB ? kHB / d->H * d->H : kRB;   // (all 16 lanes are rows: the bands of a stack have no neighbours)
  // (a longer checkpoint interval is for grids whose snapshots weigh: images are not stacked then, nor are the states
  // of a channel split over lanes, and every schedule left runs m2d_bwd_kernel, the one kernel that replays)
  g.ck_shift = d->ckpt_interval == 16 ? 2 : (d->ckpt_interval == 8 ? 1 : 0);
  // bf16 tensors with fp32 snapshots: a snapshot every 4 steps, the whole-state kernels in workgroups of 4 sweeping
  // waves (the only ones with registers to spare for quads twice as wide), one stream per image or the linked sweep
  g.snap32 = (d->flags & M2D_FLAG_FP32_SNAPSHOTS) && d->dtype == M2D_BF16;
  if (d->H <= kHB && d->B >= 2 && g.ck_shift == 0 && !g.snap32) {
    const int S = d->W > 7 ? d->W : 7;
    int64_t best = -1;
    for (int ips = 1; ips <= 64 && ips <= d->B; ++ips) {
      if ((int64_t)ips * d->H * d->W * d->E >= ((int64_t)1 << 30)) break;   // a stack is addressed like one image
      const int vB = (d->B + ips - 1) / ips;
      const int nb = (ips * d->H + rb_stacked - 1) / rb_stacked;
      const int64_t rounds = ((int64_t)vB * groups + ncu - 1) / ncu;
      const int64_t cost = rounds * ((nb - 1) * S + d->W + d->H + 8);
      if (best < 0 || cost < best) { best = cost; g.ips = ips; }
    }
    if (g.ips > 1) {
      g.stacked = true;
      g.rb = rb_stacked;
      g.vB = (d->B + g.ips - 1) / g.ips;
      g.vH = g.ips * d->H;
    }
  }
  const int B = g.vB, H = g.vH;   // what the kernels sweep
  g.nbands = (H + g.rb - 1) / g.rb;
  g.rows_last = H - (g.nbands - 1) * g.rb;
  // A band's ghost reads the row that the band before stored S - 14 steps earlier, one block
  // ahead of its use: S - 14 >= 12 steps cover the store, the block-end barrier and the staging.
  // Wide grids run the bands back to back (S = W); narrow ones are padded.  Stacked images have no
  // such dependence.
  if (g.stacked) {
    g.S = d->W > 7 ? d->W : 7;
    g.T_total = (g.nbands - 1) * g.S + d->W + d->H;   // (the rows of an image trail its first row: skew_row)
  } else {
    g.S = (g.nbands > 1 && d->W >= 26) ? d->W : (d->W + kHB - 1 > 26 ? d->W + kHB - 1 : 26);
    g.T_total = (g.nbands - 1) * g.S + d->W + g.rows_last;
  }
  g.nblk = (g.T_total + kCK - 1) / kCK;
  // Few images with many bands leave most of the device idle when each image is one sequential
  // stream.  Then every band gets workgroups of its own (a padded stream, one window of S steps
  // per band), all in one launch, and band k trails band k-1 by kLinkLag blocks of steps.
  // (two or three bands: only where a band is much longer than the 28 steps by which a band trails its neighbour)
  g.sliced = !g.stacked && (g.nbands >= 4 || (g.nbands >= 2 && d->W >= 64)) && (int64_t)B * groups <= ncu / 4;
  if (g.sliced && g.nbands == 4) {
    // Four bands (more bands favour the linked sweep again: 84x84 measured) and a batch that fills half the device with workgroups of 4 waves, but not with
    // every band under way on workgroups of its own: one stream per image on workgroups of 4 waves
    // is then the faster schedule (56x56, 64 images of 32 channels: 0.99 -> 0.93 ms forward+backward).
    int s_sl = (d->W + kHB - 1 + kCK - 1) / kCK * kCK;
    if (s_sl < 28) s_sl = 28;
    const int64_t lagged = (s_sl / kCK + kLinkLag) / (kLinkLag + 1);   // bands whose windows overlap in time (a block more for the polling)
    const int64_t under_way = lagged < g.nbands ? lagged : g.nbands;
    const int64_t half = (int64_t)B * ((d->E + kFwdHalfWaves * g.CS - 1) / (kFwdHalfWaves * g.CS));
    if (half > (int64_t)B * groups && half <= ncu && half >= ncu / 2 && half * under_way > ncu) g.sliced = false;
  }
  g.nbb = 0;
  if (g.sliced) {
    g.S = (d->W + kHB - 1 + kCK - 1) / kCK * kCK;
    if (g.S < 28) g.S = 28;
    g.nbb = g.S / kCK;
    g.T_total = g.nbands * g.S;
    g.nblk = g.nbands * g.nbb;
  }
  // forward: two channels per lane where that saves rounds of workgroups (one workgroup per compute
  // unit at a time, 256 units) and the two staging buffers of such a workgroup fit the LDS (bf16
  // operands only).  A sweep with two channels per lane takes about 1.8 times
  // as long as one with a single channel (measured: 1.6 at 28x28, 2.0 at 56x56), so it pays only
  // when it at least halves the rounds: 128 channels x 128 images, not 32 channels x 256 images
  // (where half of every workgroup would idle).
  // (fp32 operands: such a kernel would need more registers than a lane has, and is not built)
  const size_t lds_ec2 = d->dtype == M2D_BF16 ? fwd_lds_bytes<bf16_t, 2>() : kLdsPerWorkgroup + 1;
  const int64_t wg1 = (int64_t)B * ((d->E + kFwdWaves * g.CS - 1) / (kFwdWaves * g.CS));
  const int64_t wg2 = (int64_t)B * ((d->E + kFwdWaves * g.CS * 2 - 1) / (kFwdWaves * g.CS * 2));
  const bool ec2 = (d->E % 2 == 0) && lds_ec2 <= kLdsPerWorkgroup && 18 * ((wg2 + ncu - 1) / ncu) < 10 * ((wg1 + ncu - 1) / ncu);
  g.fwd_ec = ec2 ? 2 : 1;
  // forward of a small batch in one stream per image: workgroups of 4 waves (16 channels) where those
  // are more than the workgroups of 8 and still no more than the compute units
  const int64_t wg_half = (int64_t)B * ((d->E + kFwdHalfWaves * g.CS - 1) / (kFwdHalfWaves * g.CS));
  // (in the linked sweep the windows of about nbb / (kLinkLag + 1) bands overlap in time: the lag and a block for the polling)
  const int64_t together = g.sliced ? ((g.nbb + kLinkLag) / (kLinkLag + 1) < g.nbands ? (g.nbb + kLinkLag) / (kLinkLag + 1) : g.nbands) : 1;
  // (a linked sweep may exceed the units by a few workgroups while most bands are under way: its start
  // and its end, with fewer bands, still gain)
  const int64_t room = g.sliced ? ncu + ncu / 16 : ncu;
  g.fwd_nw = (!g.stacked && !ec2 && wg_half > wg1 && wg_half * together <= room) ? kFwdHalfWaves : kFwdWaves;
  g.fwd_bpb = (d->E + g.fwd_nw * g.CS * g.fwd_ec - 1) / (g.fwd_nw * g.CS * g.fwd_ec);
  g.fwd_wpb = g.fwd_bpb * g.fwd_nw;
  // Few waves under way (a wave per 4 channels, the bands of a linked sweep that overlap in time): fewer
  // than three for every four SIMDs.  Then a wave per channel, each with a quarter of the states.
  const int64_t waves_whole = (int64_t)B * ((d->E + g.CS - 1) / g.CS) * together;
  const bool may_split = !g.stacked && !(d->flags & M2D_FLAG_WHOLE_STATES) && g.ck_shift == 0;
  // One stream per image: only while the workgroups of 8 channels all run at once.  The backward has a compute unit to
  // itself, so one workgroup more than units is a second round of them, and the whole-state kernels in workgroups of 4
  // waves are then ahead (B=33..48 at 56x56x64 bf16: forward+backward kernels 0.85 -> 0.76 ms; B=32: 0.48 against 0.76).
  const bool few_enough = waves_whole <= 3 * ncu && (g.sliced || (int64_t)B * ((d->E + kSplitWaves - 1) / kSplitWaves) <= ncu);
  g.fwd_split = may_split && ((d->flags & M2D_FLAG_SPLIT_STATES) || few_enough);
  // Workgroups of 8 waves (8 channels) under way on at most half of the compute units: workgroups of 4 then run on
  // twice as many, each wave with a SIMD to itself (a sweep of few images is as fast as one wave gets through its
  // blocks).
  // Both sizes of workgroup have 4 more waves that stage for them (split_helpers).  In the linked sweep workgroups of
  // 4 stay ahead up to 7 of them under way for every 5 units (measured, E=64 fp32, forward+backward kernels with
  // workgroups of 4 against 8: 384x384 1.65 against 1.86 ms, 512x512 2.56 against 2.61, 640x640 3.63 against 3.29,
  // 768x768 5.08 against 4.10).
  const int64_t wg4 = (int64_t)B * ((d->E + kSplitHalfWaves - 1) / kSplitHalfWaves) * together;
  // (one stream per image: workgroups of 4 only while each has a compute unit)
  const int split_nw = (g.sliced ? 5 * wg4 <= 7 * ncu : wg4 <= ncu) ? kSplitHalfWaves : kSplitWaves;
  if (g.fwd_split) {
    g.fwd_ec = 1;
    g.fwd_nw = split_nw;
    g.fwd_bpb = (d->E + split_nw - 1) / split_nw;
    g.fwd_wpb = g.fwd_bpb * g.fwd_nw;
  }
  g.bwd_nw = (!g.stacked && wg_half > (int64_t)B * groups && wg_half * together <= room) ? kFwdHalfWaves : kBwdWaves;
  g.bwd_bpb = (d->E + g.bwd_nw * g.CS - 1) / (g.bwd_nw * g.CS);
  g.bwd_wpb = g.bwd_bpb * g.bwd_nw;
  // (the backward keeps one set of channel sums per workgroup of an image: with 8 channels per workgroup
  // that memory is bounded here unless the caller insists)
  const size_t split_part = sizeof(float) * (size_t)((d->E + split_nw - 1) / split_nw) * 3 * kN * (size_t)d->B * d->H * d->W;
  g.bwd_split = may_split && ((d->flags & M2D_FLAG_SPLIT_STATES) || (few_enough && split_part <= ((size_t)2 << 30)));
  if (g.bwd_split) {
    g.bwd_nw = split_nw;
    g.bwd_bpb = (d->E + split_nw - 1) / split_nw;
    g.bwd_wpb = g.bwd_bpb * g.bwd_nw;
  }
  if (g.snap32) {
    g.fwd_split = g.bwd_split = false;
    g.fwd_ec = 1;
    g.fwd_nw = g.bwd_nw = kFwdHalfWaves;
    g.fwd_bpb = g.bwd_bpb = (d->E + kFwdHalfWaves * g.CS - 1) / (kFwdHalfWaves * g.CS);
    g.fwd_wpb = g.bwd_wpb = g.fwd_bpb * kFwdHalfWaves;
  }
  g.stage_x = (d->E % (d->dtype == M2D_BF16 ? 8 : 4)) == 0;
  const size_t P = (size_t)d->B * d->H * d->W;
  g.prep_bytes = align_up(sizeof(float) * (kZeroFloats + (size_t)2 * d->E * kN + d->E));
  g.packed_bc = (d->flags & M2D_FLAG_PACKED_BC) != 0;   // the caller brings the records: nothing to reserve
  // (16-bit tensors are widened inside the scan kernels, nothing to reserve either)
  g.bc_bytes = (g.packed_bc || d->dtype == M2D_BF16) ? 0 : align_up(sizeof(float) * P * 48);
  const int every = 1 << g.ck_shift;
  g.ck_pb = g.sliced ? (g.nbb + every - 1) / every : 0;
  g.ck_nblk = g.sliced ? g.nbands * g.ck_pb : (g.nblk + every - 1) / every;
  // A snapshot every 2 steps, for the backward kernel that recomputes one step in two: where every image (or stack)
  // is one stream and a lane holds all states of its channel.  Other schedules keep one every 4 steps.
  g.ck_half = (d->ckpt_interval == 2 || d->ckpt_interval == 0) && !g.sliced && !g.fwd_split && !g.bwd_split && !g.snap32;
  if (g.ck_half) g.ck_nblk = 2 * g.nblk + 1;   // before the steps 0 and 2 of every block, and behind the last block
  g.ckpt_diag_bytes = align_up((d->dtype == M2D_BF16 && !g.snap32 ? 2 : sizeof(float)) * (size_t)B * g.ck_nblk * d->E * kN * g.HB);   // (16-bit tensors: bf16 snapshots unless fp32 ones are asked for)
  const size_t bwd_wgs = (size_t)(g.sliced ? g.nbands : 1) * B * g.bwd_bpb;
  g.ring_bytes = g.ck_shift ? align_up((d->dtype == M2D_BF16 ? 2 : sizeof(float)) * bwd_wgs * (every - 1) * g.bwd_nw * g.CS * kN * g.HB) : 0;
  const bool rows = g.nbands > 1 && !g.stacked;   // boundary rows travel between bands
  g.top_bytes = rows ? align_up(sizeof(float) * (size_t)(g.nbands - 1) * B * d->W * d->E * kN) : 0;
  g.bot_bytes = rows ? align_up(sizeof(float) * (size_t)(g.sliced ? g.nbands : 1) * B * d->W * d->E * kN) : 0;
  const size_t chains = (size_t)B * (g.fwd_bpb > g.bwd_bpb ? g.fwd_bpb : g.bwd_bpb);
  g.link_bytes = g.sliced ? align_up(sizeof(uint32_t) * (64 + 2 * g.nbands * chains * kLinkStride)) : 0;
  g.part_bytes = align_up(sizeof(float) * (size_t)g.bwd_bpb * 3 * P * kN);
  const size_t slots = g.sliced ? g.nbands : 1;
  g.pa_bytes = align_up(sizeof(float) * (size_t)B * slots * d->E * 2 * kN);
  g.pd_bytes = align_up(sizeof(float) * (size_t)B * slots * d->E);
  return g;
}

// checkpoint buffer: [state snapshots][band boundary rows][packed B,C (fp32 tensors only)][set-up area]
// (the set-up area -- page of zeros, A * log2 e, D -- is the forward's: a backward that gets the buffer needs no
// set-up launch of its own, unless it has progress counts to clear)
size_t ckpt_bytes_of(const Geometry& g) { return g.ckpt_diag_bytes + g.top_bytes + g.bc_bytes + g.prep_bytes; }

size_t workspace_bytes_of(const Geometry& g, int pass, int have_ckpt) {
  size_t n = g.prep_bytes + g.link_bytes;
  if (pass == M2D_PASS_FWD) {
    if (!have_ckpt) n += g.top_bytes + g.bc_bytes;
  } else {
    n += g.part_bytes + g.pa_bytes + g.pd_bytes + g.bot_bytes + g.ring_bytes;
    if (!have_ckpt) n += ckpt_bytes_of(g);
  }
  return n;
}

bool misaligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) != 0; }

void fill_common(ScanParams& sp, const m2d_desc* d, const Geometry& g) {
  sp.B = g.vB; sp.H = g.vH; sp.W = d->W; sp.E = d->E;
  sp.stacked = g.stacked ? 1 : 0; sp.ips = g.ips; sp.Himg = d->H; sp.Breal = d->B; sp.Hs = g.vH;
  sp.Ptot = (int64_t)d->B * d->H * d->W;
  sp.nbands = g.nbands; sp.nblk = g.nblk;
  sp.S = g.S; sp.T_total = g.T_total; sp.rows_last = g.rows_last; sp.rb = g.rb;
  sp.magicS = (uint32_t)(((uint64_t)1 << 32) / (uint64_t)g.S);
  sp.sliced = g.sliced ? 1 : 0; sp.sl_nbb = g.nbb;
  sp.pa_slots = g.sliced ? g.nbands : 1;
  sp.bot_stride = g.sliced ? (int64_t)g.vB * d->W * d->E * kN : 0;
  sp.flip = (d->flags & M2D_FLAG_FLIP) ? 1 : 0;
  sp.dpre = (d->flags & M2D_FLAG_DPRE) ? 1 : 0;
  sp.ck_shift = g.ck_shift; sp.ck_pb = g.ck_pb; sp.ck_nblk = g.ck_nblk; sp.ck_half = g.ck_half ? 1 : 0;
  sp.ring = nullptr;
}

// A kernel that needs more than 64 KB of dynamic LDS has to be told so once per device (each
// device loads its own copy of the code object).  `seen` holds one bit per device ordinal.
inline bool allow_dynamic_lds(const void* kernel, size_t bytes, std::atomic<uint64_t>& seen) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return false;
  const uint64_t bit = 1ull << (dev & 63);
  if (seen.load(std::memory_order_relaxed) & bit) return true;
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess) return false;
  seen.fetch_or(bit, std::memory_order_relaxed);
  return true;
}

// Set-up area: [page of zeros][A_T*log2e][A_L*log2e][D], all fp32.
template <typename T>
int launch_prep(ScanParams& sp, const m2d_desc* d, const Geometry& g, const void* AT, const void* AL, const void* D, float* base,
                uint32_t* link_words, hipStream_t st, bool ready = false) {
  const int n_link = (int)(g.link_bytes / sizeof(uint32_t));
  sp.link_err = link_words;   // (the first 64 words: the error word; then forward counts, then backward counts)
  float* zeros = base;
  float* A2T = base + kZeroFloats;
  float* A2L = A2T + (size_t)d->E * kN;
  float* Df = A2L + (size_t)d->E * kN;
  sp.zeros = zeros; sp.A2T = A2T; sp.A2L = A2L; sp.Df = Df;
  if (ready && n_link == 0) return M2D_OK;   // the forward of this problem filled the area, and there is nothing to clear
  const int n = d->E * kN > kZeroFloats ? d->E * kN : kZeroFloats;
  if (d->flags & M2D_FLAG_RAW_PARAMS)
    hipLaunchKernelGGL((m2d_prep_kernel<T, true>), dim3((n + 255) / 256), dim3(256), 0, st, AT, AL, D, zeros, A2T, A2L, Df, d->E, link_words, n_link);
  else
    hipLaunchKernelGGL((m2d_prep_kernel<T, false>), dim3((n + 255) / 256), dim3(256), 0, st, AT, AL, D, zeros, A2T, A2L, Df, d->E, link_words, n_link);
  return hipGetLastError() == hipSuccess ? M2D_OK : M2D_ERR_HIP;
}

// Points sp.bt/bl/cc at the packed fp32 copy of B_T, B_L, C (made here unless `ready`, or brought
// by the caller in place of B_T).
template <typename T>
int stage_bc(ScanParams& sp, const m2d_desc* d, const void* BT, const void* BL, const void* C, float* wide,
             bool ready, hipStream_t st) {
  if (d->flags & M2D_FLAG_PACKED_BC) { wide = static_cast<float*>(const_cast<void*>(BT)); ready = true; }
  sp.bt = wide; sp.bl = wide + kN; sp.cc = wide + 2 * kN;
  sp.bc_stride = 48;
  if (ready) return M2D_OK;
  const int64_t P = (int64_t)d->B * d->H * d->W;
  hipLaunchKernelGGL(m2d_pack_bc_kernel<T>, dim3((unsigned)((P * 3 + 255) / 256)), dim3(256), 0, st,
                     static_cast<const T*>(BT), static_cast<const T*>(BL), static_cast<const T*>(C), wide, P);
  return hipGetLastError() == hipSuccess ? M2D_OK : M2D_ERR_HIP;
}

// Development aid: -DM2D_QUICK=1 builds only the kernels of many 16-bit images in one stream each, in workgroups of
// 8 waves (a twentieth of the compile time), -DM2D_QUICK=2 (3) only the linked sweep of fp32 (16-bit) images in workgroups of 4 waves;
// every other problem then answers M2D_ERR_UNSUPPORTED.
#if defined(M2D_QUICK) && M2D_QUICK >= 2 && M2D_QUICK <= 3
#define M2D_BUILT(T, SX, MODE, NW, OTHER) (sizeof(T) == (M2D_QUICK == 3 ? 2 : 4) && (MODE) == kModeSliced && (NW) == 4)
#elif defined(M2D_QUICK)
#define M2D_BUILT(T, SX, MODE, NW, OTHER) (sizeof(T) == 2 && (SX) && (MODE) == kModeSweep && (NW) == (M2D_QUICK == 1 ? 8 : 4) && (OTHER))
#else
#define M2D_BUILT(T, SX, MODE, NW, OTHER) true
#endif

template <typename T, int EC, bool CK, bool WY, bool SX, int MODE, int NW, bool HALF = false, typename ST = T>
int launch_fwd_as(const ScanParams& sp, hipStream_t st) {
  if constexpr (!M2D_BUILT(T, SX, MODE, NW, EC == 1)) return M2D_ERR_UNSUPPORTED; else {
  constexpr size_t lds = fwd_lds_bytes<T, EC, NW>();
  if (lds > kLdsPerWorkgroup) return M2D_ERR_UNSUPPORTED;   // (make_geometry never picks such a layout)
  static std::atomic<uint64_t> seen{0};
  if (!allow_dynamic_lds(reinterpret_cast<const void*>(&m2d_fwd_kernel<T, EC, CK, WY, SX, MODE, NW, HALF, ST>), lds, seen)) return M2D_ERR_HIP;
  hipLaunchKernelGGL((m2d_fwd_kernel<T, EC, CK, WY, SX, MODE, NW, HALF, ST>), dim3((unsigned)sp.nwg), dim3((NW + whole_helpers<MODE, NW, EC>()) * 64), lds, st, sp);
  return hipGetLastError() == hipSuccess ? M2D_OK : M2D_ERR_HIP;
  }
}

template <typename T, int NWS = kSplitWaves>
constexpr size_t fwd_split_lds_bytes() { return 2 * (size_t)Stage<T, 3, NWS, false>::kBytes + (sizeof(T) == 2 ? 2 * kRawBytes : 0); }
template <typename T, bool CK, bool WY, bool SX, int MODE, int NWS = kSplitWaves>
int launch_fwd_split_as(const ScanParams& sp, hipStream_t st) {
  if constexpr (!M2D_BUILT(T, SX, MODE, NWS, false)) return M2D_ERR_UNSUPPORTED; else {
  constexpr size_t lds = fwd_split_lds_bytes<T, NWS>();
  static_assert(lds <= kLdsPerWorkgroup, "staging must fit the LDS");
  static std::atomic<uint64_t> seen{0};
  if (!allow_dynamic_lds(reinterpret_cast<const void*>(&m2d_fwd_split_kernel<T, CK, WY, SX, MODE, NWS>), lds, seen)) return M2D_ERR_HIP;
  hipLaunchKernelGGL((m2d_fwd_split_kernel<T, CK, WY, SX, MODE, NWS>), dim3((unsigned)sp.nwg), dim3((NWS + split_helpers<MODE, NWS, SX>()) * 64), lds, st, sp);
  return hipGetLastError() == hipSuccess ? M2D_OK : M2D_ERR_HIP;
  }
}
// (x and deltas of a workgroup's channels are one or two 16-byte chunks per cell, or 4 channels of a 16-bit tensor half of one)
template <typename T, int MODE>
int launch_fwd_split(const ScanParams& sp, bool stage_x, bool ckpt, bool write_y, hipStream_t st, int nw = kSplitWaves) {
  if (nw == kSplitHalfWaves) {
    if (stage_x) {
      if (ckpt && write_y) return launch_fwd_split_as<T, true, true, true, MODE, kSplitHalfWaves>(sp, st);
      if (ckpt) return launch_fwd_split_as<T, true, false, true, MODE, kSplitHalfWaves>(sp, st);
      return launch_fwd_split_as<T, false, true, true, MODE, kSplitHalfWaves>(sp, st);
    }
    if (ckpt && write_y) return launch_fwd_split_as<T, true, true, false, MODE, kSplitHalfWaves>(sp, st);
    if (ckpt) return launch_fwd_split_as<T, true, false, false, MODE, kSplitHalfWaves>(sp, st);
    return launch_fwd_split_as<T, false, true, false, MODE, kSplitHalfWaves>(sp, st);
  }
  if (stage_x) {
    if (ckpt && write_y) return launch_fwd_split_as<T, true, true, true, MODE>(sp, st);
    if (ckpt) return launch_fwd_split_as<T, true, false, true, MODE>(sp, st);
    return launch_fwd_split_as<T, false, true, true, MODE>(sp, st);
  }
  if (ckpt && write_y) return launch_fwd_split_as<T, true, true, false, MODE>(sp, st);
  if (ckpt) return launch_fwd_split_as<T, true, false, false, MODE>(sp, st);
  return launch_fwd_split_as<T, false, true, false, MODE>(sp, st);
}

template <typename T, int EC, bool SX, int MODE, int NW = kFwdWaves>
int launch_fwd_mode(const ScanParams& sp, bool ckpt, bool write_y, hipStream_t st) {
  if constexpr (MODE != kModeSliced) {
    if (ckpt && sp.ck_half) return write_y ? launch_fwd_as<T, EC, true, true, SX, MODE, NW, true>(sp, st) : launch_fwd_as<T, EC, true, false, SX, MODE, NW, true>(sp, st);
  }
  if (ckpt && write_y) return launch_fwd_as<T, EC, true, true, SX, MODE, NW>(sp, st);
  if (ckpt) return launch_fwd_as<T, EC, true, false, SX, MODE, NW>(sp, st);
  return launch_fwd_as<T, EC, false, true, SX, MODE, NW>(sp, st);
}

template <typename T>
int launch_fwd(const ScanParams& sp0, const m2d_desc* d, const Geometry& g, bool ckpt, bool write_y, hipStream_t st) {
  ScanParams sp = sp0;
  sp.bpb = g.fwd_bpb;
  sp.nwg = g.vB * g.fwd_bpb;
  auto once = [&]() {
    if constexpr (sizeof(T) == 2) {
      if (g.snap32 && ckpt) {   // bf16 tensors, fp32 snapshots: the forward that keeps them (for the caller, or rebuilt inside the backward)
        if (g.sliced) {
          if (g.stage_x) return write_y ? launch_fwd_as<T, 1, true, true, true, kModeSliced, kFwdHalfWaves, false, float>(sp, st) : launch_fwd_as<T, 1, true, false, true, kModeSliced, kFwdHalfWaves, false, float>(sp, st);
          return write_y ? launch_fwd_as<T, 1, true, true, false, kModeSliced, kFwdHalfWaves, false, float>(sp, st) : launch_fwd_as<T, 1, true, false, false, kModeSliced, kFwdHalfWaves, false, float>(sp, st);
        }
        if (g.stage_x) return write_y ? launch_fwd_as<T, 1, true, true, true, kModeSweep, kFwdHalfWaves, false, float>(sp, st) : launch_fwd_as<T, 1, true, false, true, kModeSweep, kFwdHalfWaves, false, float>(sp, st);
        return write_y ? launch_fwd_as<T, 1, true, true, false, kModeSweep, kFwdHalfWaves, false, float>(sp, st) : launch_fwd_as<T, 1, true, false, false, kModeSweep, kFwdHalfWaves, false, float>(sp, st);
      }
    }
    if (g.fwd_split)
      return g.sliced ? launch_fwd_split<T, kModeSliced>(sp, g.stage_x, ckpt, write_y, st, g.fwd_nw)
                      : launch_fwd_split<T, kModeSweep>(sp, g.stage_x, ckpt, write_y, st, g.fwd_nw);
    if (g.sliced) {   // (the linked sweep is only chosen where one channel per lane is)
      if (g.fwd_nw == kFwdHalfWaves)
        return g.stage_x ? launch_fwd_mode<T, 1, true, kModeSliced, kFwdHalfWaves>(sp, ckpt, write_y, st)
                         : launch_fwd_mode<T, 1, false, kModeSliced, kFwdHalfWaves>(sp, ckpt, write_y, st);
      return g.stage_x ? launch_fwd_mode<T, 1, true, kModeSliced>(sp, ckpt, write_y, st) : launch_fwd_mode<T, 1, false, kModeSliced>(sp, ckpt, write_y, st);
    }
    if (g.stacked) {
      if constexpr (sizeof(T) == 2)   // (fp32 operands of two channels per lane do not fit the LDS: never chosen, not built)
      if (g.fwd_ec == 2)
        return g.stage_x ? launch_fwd_mode<T, 2, true, kModeStacked>(sp, ckpt, write_y, st) : launch_fwd_mode<T, 2, false, kModeStacked>(sp, ckpt, write_y, st);
      return g.stage_x ? launch_fwd_mode<T, 1, true, kModeStacked>(sp, ckpt, write_y, st) : launch_fwd_mode<T, 1, false, kModeStacked>(sp, ckpt, write_y, st);
    }
    if constexpr (sizeof(T) == 2)
    if (g.fwd_ec == 2)
      return g.stage_x ? launch_fwd_mode<T, 2, true, kModeSweep>(sp, ckpt, write_y, st) : launch_fwd_mode<T, 2, false, kModeSweep>(sp, ckpt, write_y, st);
    if (g.fwd_nw == kFwdHalfWaves)
      return g.stage_x ? launch_fwd_mode<T, 1, true, kModeSweep, kFwdHalfWaves>(sp, ckpt, write_y, st)
                       : launch_fwd_mode<T, 1, false, kModeSweep, kFwdHalfWaves>(sp, ckpt, write_y, st);
    return g.stage_x ? launch_fwd_mode<T, 1, true, kModeSweep>(sp, ckpt, write_y, st) : launch_fwd_mode<T, 1, false, kModeSweep>(sp, ckpt, write_y, st);
  };
  if (g.sliced) {   // every band on workgroups of its own, band 0 first: a band waits for the one before it
    sp.nwg = g.nbands * g.vB * g.fwd_bpb;
    sp.prog = sp.link_err + 64;
  }
  return once();
}

template <typename T>
int run_fwd(const m2d_desc* d, const Geometry& g, ScanParams sp, const void* AT, const void* AL, const void* BT,
            const void* BL, const void* C, const void* D, void* ckpt, void* ws, hipStream_t st) {
  char* w = static_cast<char*>(ws);
  float* prep = reinterpret_cast<float*>(w);
  w += g.prep_bytes;
  uint32_t* link_words = reinterpret_cast<uint32_t*>(w); w += g.link_bytes;
  char* keep = ckpt ? static_cast<char*>(ckpt) + g.ckpt_diag_bytes : w;   // [top][packed B,C]
  sp.ckpt = ckpt ? static_cast<float*>(ckpt) : nullptr;
  sp.top = reinterpret_cast<float*>(keep);
  if (ckpt) prep = reinterpret_cast<float*>(keep + g.top_bytes + g.bc_bytes);   // kept for the backward
  int rc = launch_prep<T>(sp, d, g, AT, AL, D, prep, link_words, st);
  if (rc) return rc;
  if ((!ckpt || sizeof(T) == 2) && !g.packed_bc) {   // the kernel takes the tensors as they are (fp32: only where no backward will want the packed copy)
    sp.bcd[0] = BT; sp.bcd[1] = BL; sp.bcd[2] = C; sp.bcd[3] = BT;
    sp.bt = sp.bl = sp.cc = nullptr;
    sp.bc_stride = 0;
    sp.bc_direct = 1;
  } else {
    rc = stage_bc<T>(sp, d, BT, BL, C, reinterpret_cast<float*>(keep + g.top_bytes), false, st);
  }
  if (rc) return rc;
  if ((d->flags & M2D_FLAG_TEST_DEAD_LINK) && g.sliced && g.nbands >= 2) sp.link_test = 1 + 1;   // the second band's neighbour never reports
  if (g_profile) (void)hipEventRecord(g_ev[M2D_PASS_FWD][0], st);
  rc = launch_fwd<T>(sp, d, g, ckpt != nullptr, true, st);
  if (g_profile) (void)hipEventRecord(g_ev[M2D_PASS_FWD][1], st);
  return rc;
}

template <typename T, bool SX, int MODE, int NW, bool REPLAY = false, typename ST = T>
int launch_bwd_as(const ScanParams& sp, hipStream_t st) {
  if constexpr (!M2D_BUILT(T, SX, MODE, NW, !REPLAY)) return M2D_ERR_UNSUPPORTED; else {
  constexpr size_t lds = bwd_lds_bytes<T, NW>();
  static std::atomic<uint64_t> seen{0};
  if (!allow_dynamic_lds(reinterpret_cast<const void*>(&m2d_bwd_kernel<T, SX, MODE, NW, REPLAY, ST>), lds, seen)) return M2D_ERR_HIP;
  hipLaunchKernelGGL((m2d_bwd_kernel<T, SX, MODE, NW, REPLAY, ST>), dim3((unsigned)sp.nwg), dim3((NW + (REPLAY ? 0 : whole_helpers<MODE, NW>())) * 64), lds, st, sp);
  return hipGetLastError() == hipSuccess ? M2D_OK : M2D_ERR_HIP;
  }
}

template <typename T, int NW>
constexpr size_t bwd2_lds_bytes() {
  return sizeof(float2) * bwd2_exchange_sets<T, NW>() * NW * 3 * 64 + sizeof(float) * NW * 4 * 2 * kN + 256 +
         2 * (size_t)Stage<T, 4, NW * 4, true>::kBytes + (sizeof(T) == 2 ? 2 * kRawBytes : 0);
}
template <typename T, bool SX, int MODE, int NW>
int launch_bwd2_as(const ScanParams& sp, hipStream_t st) {
  if constexpr (!M2D_BUILT(T, SX, MODE, NW, true)) return M2D_ERR_UNSUPPORTED; else {
  constexpr size_t lds = bwd2_lds_bytes<T, NW>();
  static_assert(lds <= kLdsPerWorkgroup, "exchange sets and staging must fit the LDS");
  static std::atomic<uint64_t> seen{0};
  if (!allow_dynamic_lds(reinterpret_cast<const void*>(&m2d_bwd2_kernel<T, SX, MODE, NW>), lds, seen)) return M2D_ERR_HIP;
  hipLaunchKernelGGL((m2d_bwd2_kernel<T, SX, MODE, NW>), dim3((unsigned)sp.nwg), dim3((NW + whole_helpers<MODE, NW>()) * 64), lds, st, sp);
  return hipGetLastError() == hipSuccess ? M2D_OK : M2D_ERR_HIP;
  }
}

template <typename T, int NWS = kSplitWaves>
constexpr size_t bwd_split_lds_bytes() {
  return sizeof(float4) * 2 * NWS * 3 * 64 + 2 * (size_t)Stage<T, 4, NWS, true>::kBytes + (sizeof(T) == 2 ? 2 * kRawBytes : 0);
}
template <typename T, bool SX, int MODE, int NWS = kSplitWaves>
int launch_bwd_split_as(const ScanParams& sp, hipStream_t st) {
  if constexpr (!M2D_BUILT(T, SX, MODE, NWS, false)) return M2D_ERR_UNSUPPORTED; else {
  constexpr size_t lds = bwd_split_lds_bytes<T, NWS>();
  static_assert(lds <= kLdsPerWorkgroup, "exchange buffers and staging must fit the LDS");
  static std::atomic<uint64_t> seen{0};
  if (!allow_dynamic_lds(reinterpret_cast<const void*>(&m2d_bwd_split_kernel<T, SX, MODE, NWS>), lds, seen)) return M2D_ERR_HIP;
  hipLaunchKernelGGL((m2d_bwd_split_kernel<T, SX, MODE, NWS>), dim3((unsigned)sp.nwg), dim3((NWS + split_helpers<MODE, NWS, SX>()) * 64), lds, st, sp);
  return hipGetLastError() == hipSuccess ? M2D_OK : M2D_ERR_HIP;
  }
}
template <typename T, int MODE>
int launch_bwd_split(const ScanParams& sp, bool stage_x, hipStream_t st, int nw = kSplitWaves) {
  if (nw == kSplitHalfWaves)
    return stage_x ? launch_bwd_split_as<T, true, MODE, kSplitHalfWaves>(sp, st) : launch_bwd_split_as<T, false, MODE, kSplitHalfWaves>(sp, st);
  return stage_x ? launch_bwd_split_as<T, true, MODE>(sp, st) : launch_bwd_split_as<T, false, MODE>(sp, st);
}

template <typename T, bool SX, int MODE>
int launch_bwd(const ScanParams& sp, hipStream_t st, int nw = kBwdWaves, bool snap32 = false) {
  if constexpr (sizeof(T) == 2 && MODE != kModeStacked) {
    if (snap32) return launch_bwd_as<T, SX, MODE, kFwdHalfWaves, false, float>(sp, st);   // bf16 tensors, fp32 snapshots
  }
  if constexpr (MODE != kModeSliced) {
    if (sp.ck_half) {   // snapshots every 2 steps
      if constexpr (MODE != kModeStacked) { if (nw == kFwdHalfWaves) return launch_bwd2_as<T, SX, MODE, kFwdHalfWaves>(sp, st); }
      return launch_bwd2_as<T, SX, MODE, kBwdWaves>(sp, st);
    }
  }
  if constexpr (MODE != kModeStacked) {
    if (sp.ck_shift > 0)   // a longer checkpoint interval: the kernel that replays the forward between snapshots
      return nw == kFwdHalfWaves ? launch_bwd_as<T, SX, MODE, kFwdHalfWaves, true>(sp, st) : launch_bwd_as<T, SX, MODE, kBwdWaves, true>(sp, st);
    if (nw == kFwdHalfWaves) return launch_bwd_as<T, SX, MODE, kFwdHalfWaves>(sp, st);
  }
  return launch_bwd_as<T, SX, MODE, kBwdWaves>(sp, st);
}

template <typename T>
int run_bwd(const m2d_desc* d, const Geometry& g, ScanParams sp, const void* AT, const void* AL, const void* BT,
            const void* BL, const void* C, const void* D, const void* ckpt, void* dAT, void* dAL, void* dBT,
            void* dBL, void* dC, void* dD, void* ws, hipStream_t st) {
  char* w = static_cast<char*>(ws);
  float* prep = reinterpret_cast<float*>(w); w += g.prep_bytes;
  uint32_t* link_words = reinterpret_cast<uint32_t*>(w); w += g.link_bytes;
  sp.part = reinterpret_cast<float*>(w); w += g.part_bytes;
  if (d->flags & M2D_FLAG_SUM_PARTS) sp.part = static_cast<float*>(dBT);   // the per-workgroup channel sums go to the caller, as they are
  sp.pA = reinterpret_cast<float*>(w); w += g.pa_bytes;
  sp.pD = reinterpret_cast<float*>(w); w += g.pd_bytes;
  sp.bot = reinterpret_cast<float*>(w); w += g.bot_bytes;
  sp.ring = w; w += g.ring_bytes;
  char* ck = ckpt ? const_cast<char*>(static_cast<const char*>(ckpt)) : w;
  if (ckpt) prep = reinterpret_cast<float*>(ck + g.ckpt_diag_bytes + g.top_bytes + g.bc_bytes);   // as the forward left it
  int rc = launch_prep<T>(sp, d, g, AT, AL, D, prep, link_words, st, ckpt != nullptr);
  if (rc) return rc;
  sp.ckpt = reinterpret_cast<float*>(ck);
  sp.top = reinterpret_cast<float*>(ck + g.ckpt_diag_bytes);
  if (sizeof(T) == 2 && !g.packed_bc) {   // widened inside the kernels (also by the forward sweep below)
    sp.bcd[0] = BT; sp.bcd[1] = BL; sp.bcd[2] = C; sp.bcd[3] = BT;
    sp.bt = sp.bl = sp.cc = nullptr;
    sp.bc_stride = 0;
    sp.bc_direct = 1;
  } else {
    rc = stage_bc<T>(sp, d, BT, BL, C, reinterpret_cast<float*>(ck + g.ckpt_diag_bytes + g.top_bytes), ckpt != nullptr, st);
  }
  if (rc) return rc;
  if (!ckpt) {   // rebuild the checkpoints with one forward sweep that writes no y
    rc = launch_fwd<T>(sp, d, g, true, false, st);
    if (rc) return rc;
  }
  sp.bpb = g.bwd_bpb;
  sp.nwg = g.vB * g.bwd_bpb;
  if ((d->flags & M2D_FLAG_TEST_DEAD_LINK) && g.sliced && g.nbands >= 2) sp.link_test = 1 + (g.nbands - 2);   // the last band but one waits for the last
  if (g_profile) (void)hipEventRecord(g_ev[M2D_PASS_BWD][0], st);
  if (!g.sliced) {
    if (g.bwd_split) rc = launch_bwd_split<T, kModeSweep>(sp, g.stage_x, st, g.bwd_nw);
    else if (g.stacked) rc = g.stage_x ? launch_bwd<T, true, kModeStacked>(sp, st) : launch_bwd<T, false, kModeStacked>(sp, st);
    else rc = g.stage_x ? launch_bwd<T, true, kModeSweep>(sp, st, g.bwd_nw, g.snap32) : launch_bwd<T, false, kModeSweep>(sp, st, g.bwd_nw, g.snap32);
  } else {
    // every band on workgroups of its own, the last band first: a band waits for the one below it
    sp.nwg = g.nbands * g.vB * g.bwd_bpb;
    sp.prog = sp.link_err + 64 + (size_t)g.nbands * g.vB * (g.fwd_bpb > g.bwd_bpb ? g.fwd_bpb : g.bwd_bpb) * kLinkStride;
    if (g.bwd_split) rc = launch_bwd_split<T, kModeSliced>(sp, g.stage_x, st, g.bwd_nw);
    else rc = g.stage_x ? launch_bwd<T, true, kModeSliced>(sp, st, g.bwd_nw, g.snap32) : launch_bwd<T, false, kModeSliced>(sp, st, g.bwd_nw, g.snap32);
  }
  if (g_profile) (void)hipEventRecord(g_ev[M2D_PASS_BWD][1], st);
  if (rc) return rc;
  const int64_t P = (int64_t)d->B * d->H * d->W;
  const int parts_stay = (d->flags & M2D_FLAG_SUM_PARTS) ? 1 : 0;
  const int64_t quad_blocks = parts_stay ? 0 : (3 * P * (kN / 4) + 255) / 256;
  const int64_t tail_blocks = (((int64_t)d->E * 2 * kN + d->E) * 16 + 255) / 256;   // 16 lanes per position sum
  if (d->flags & M2D_FLAG_RAW_PARAMS)
    hipLaunchKernelGGL((m2d_finalize_kernel<T, true>), dim3((unsigned)(quad_blocks + tail_blocks)), dim3(256), 0, st, sp,
                       static_cast<T*>(dC), static_cast<T*>(dBT), static_cast<T*>(dBL), dAT, dAL, dD, parts_stay);
  else
    hipLaunchKernelGGL((m2d_finalize_kernel<T, false>), dim3((unsigned)(quad_blocks + tail_blocks)), dim3(256), 0, st, sp,
                       static_cast<T*>(dC), static_cast<T*>(dBT), static_cast<T*>(dBL), dAT, dAL, dD, parts_stay);
  return hipGetLastError() == hipSuccess ? M2D_OK : M2D_ERR_HIP;
}

}  // namespace

// ---------------------------------------------------------------------------------------- C ABI
extern "C" {


int m2d_version(void) { return 700; }

const char* m2d_status_str(int status) {
  switch (status) {
    case M2D_OK: return "ok";
    case M2D_ERR_NULL_POINTER: return "null pointer argument";
    case M2D_ERR_BAD_SHAPE: return "bad shape (all dims >= 1, H >= 2, W >= 2 required)";
    case M2D_ERR_UNSUPPORTED: return "unsupported dtype, d_state, flags or image size (this build: f32/bf16, N=16, H*W < 2^24, H*W*E < 2^30)";
    case M2D_ERR_WORKSPACE: return "workspace or checkpoint buffer too small";
    case M2D_ERR_MISALIGNED: return "misaligned pointer (tensors 16 B, workspace/checkpoints 256 B)";
    case M2D_ERR_HIP: return "HIP runtime error";
    case M2D_ERR_TOO_LARGE: return "problem needs more scratch than the static buffer of m2d_scan_fwd_noalloc holds (M2D_NOALLOC_SCRATCH_BYTES)";
    default: return "unknown status";
  }
}

int m2d_desc_check(const m2d_desc* desc) { return check_desc(desc); }

int m2d_profile_enable(int on) {
  if (on && !g_ev[0][0]) {
    for (auto& pr : g_ev)
      for (auto& ev : pr)
        if (hipEventCreate(&ev) != hipSuccess) return M2D_ERR_HIP;
  }
  g_profile = on != 0;
  return M2D_OK;
}

int m2d_profile_last_ms(int pass, float* ms) {
  if (!ms) return M2D_ERR_NULL_POINTER;
  if ((pass != M2D_PASS_FWD && pass != M2D_PASS_BWD) || !g_ev[0][0]) return M2D_ERR_UNSUPPORTED;
  if (hipEventSynchronize(g_ev[pass][1]) != hipSuccess) return M2D_ERR_HIP;
  return hipEventElapsedTime(ms, g_ev[pass][0], g_ev[pass][1]) == hipSuccess ? M2D_OK : M2D_ERR_HIP;
}

size_t m2d_scan_workspace_bytes(const m2d_desc* desc, int pass, int have_ckpt) {
  if (check_desc(desc) != M2D_OK || (pass != M2D_PASS_FWD && pass != M2D_PASS_BWD)) return 0;
  return workspace_bytes_of(make_geometry(desc), pass, have_ckpt);
}

size_t m2d_scan_ckpt_bytes(const m2d_desc* desc) {
  if (check_desc(desc) != M2D_OK) return 0;
  return ckpt_bytes_of(make_geometry(desc));
}

int m2d_scan_fwd(const m2d_desc* desc, const void* x, const void* deltaT, const void* deltaL, const void* AT,
                 const void* AL, const void* BT, const void* BL, const void* C, const void* D, void* y, void* ckpt,
                 size_t ckpt_bytes, void* workspace, size_t workspace_bytes, void* stream) {
  int rc = check_desc(desc);
  if (rc) return rc;
  const bool packed = (desc->flags & M2D_FLAG_PACKED_BC) != 0;   // B_T carries the records, B_L and C are not read
  const void* req[] = {x, deltaT, deltaL, AT, AL, BT, packed ? BT : BL, packed ? BT : C, D, y, workspace};
  for (const void* q : req) if (!q) return M2D_ERR_NULL_POINTER;
  for (const void* q : req) if (misaligned(q, 16)) return M2D_ERR_MISALIGNED;
  if (misaligned(workspace, 256) || (ckpt && misaligned(ckpt, 256))) return M2D_ERR_MISALIGNED;
  const Geometry g = make_geometry(desc);
  if (workspace_bytes < workspace_bytes_of(g, M2D_PASS_FWD, ckpt != nullptr)) return M2D_ERR_WORKSPACE;
  if (ckpt && ckpt_bytes < ckpt_bytes_of(g)) return M2D_ERR_WORKSPACE;
  ScanParams sp = {};
  fill_common(sp, desc, g);
  sp.x = x; sp.dT = deltaT; sp.dL = deltaL; sp.y = y;
  hipStream_t st = static_cast<hipStream_t>(stream);
  return desc->dtype == M2D_F32 ? run_fwd<float>(desc, g, sp, AT, AL, BT, BL, C, D, ckpt, workspace, st)
                                : run_fwd<bf16_t>(desc, g, sp, AT, AL, BT, BL, C, D, ckpt, workspace, st);
}

int m2d_scan_bwd(const m2d_desc* desc, const void* x, const void* deltaT, const void* deltaL, const void* AT,
                 const void* AL, const void* BT, const void* BL, const void* C, const void* D, const void* dy,
                 const void* ckpt, size_t ckpt_bytes, void* dx, void* d_deltaT, void* d_deltaL, void* d_AT,
                 void* d_AL, void* d_BT, void* d_BL, void* d_C, void* d_D, void* workspace,
                 size_t workspace_bytes, void* stream) {
  int rc = check_desc(desc);
  if (rc) return rc;
  const bool packed = (desc->flags & M2D_FLAG_PACKED_BC) != 0;   // B_T carries the records, B_L and C are not read
  const bool parts = (desc->flags & M2D_FLAG_SUM_PARTS) != 0;   // d_BT receives the per-workgroup sums, d_BL and d_C are not written
  const void* req[] = {x, deltaT, deltaL, AT, AL, BT, packed ? BT : BL, packed ? BT : C, D, dy, dx, d_deltaT, d_deltaL,
                       d_AT, d_AL, d_BT, parts ? d_BT : d_BL, parts ? d_BT : d_C, d_D, workspace};
  for (const void* q : req) if (!q) return M2D_ERR_NULL_POINTER;
  for (const void* q : req) if (misaligned(q, 16)) return M2D_ERR_MISALIGNED;
  if (misaligned(workspace, 256) || (ckpt && misaligned(ckpt, 256))) return M2D_ERR_MISALIGNED;
  const Geometry g = make_geometry(desc);
  if (workspace_bytes < workspace_bytes_of(g, M2D_PASS_BWD, ckpt != nullptr)) return M2D_ERR_WORKSPACE;
  if (ckpt && ckpt_bytes < ckpt_bytes_of(g)) return M2D_ERR_WORKSPACE;
  ScanParams sp = {};
  fill_common(sp, desc, g);
  sp.x = x; sp.dT = deltaT; sp.dL = deltaL; sp.dy = dy;
  sp.dx = dx; sp.ddT = d_deltaT; sp.ddL = d_deltaL;
  hipStream_t st = static_cast<hipStream_t>(stream);
  return desc->dtype == M2D_F32
             ? run_bwd<float>(desc, g, sp, AT, AL, BT, BL, C, D, ckpt, d_AT, d_AL, d_BT, d_BL, d_C, d_D, workspace, st)
             : run_bwd<bf16_t>(desc, g, sp, AT, AL, BT, BL, C, D, ckpt, d_AT, d_AL, d_BT, d_BL, d_C, d_D, workspace, st);
}

int m2d_scan_sum_parts(const m2d_desc* desc) {
  if (check_desc(desc) != M2D_OK) return 0;
  return make_geometry(desc).bwd_bpb;
}

int m2d_scan_plan(const m2d_desc* desc, int pass, char* text, size_t cap) {
  if (!desc || !text) return M2D_ERR_NULL_POINTER;
  if (cap == 0 || (pass != M2D_PASS_FWD && pass != M2D_PASS_BWD)) return M2D_ERR_BAD_SHAPE;
  const int rc = check_desc(desc);
  if (rc != M2D_OK) { text[0] = 0; return rc; }
  const Geometry g = make_geometry(desc);
  const bool fwd = pass == M2D_PASS_FWD;
  const bool split = fwd ? g.fwd_split : g.bwd_split;
  const int nw = fwd ? g.fwd_nw : g.bwd_nw, bpb = fwd ? g.fwd_bpb : g.bwd_bpb;
  const int per_lane = fwd ? g.fwd_ec : 1;
  const long long wgs = (long long)(g.sliced ? g.nbands : 1) * g.vB * bpb;
  char sched[96];
  if (g.sliced) snprintf(sched, sizeof sched, "linked sweep, %d bands", g.nbands);
  else if (g.stacked) snprintf(sched, sizeof sched, "stacked images, %d per stream, %d bands", g.ips, g.nbands);
  else snprintf(sched, sizeof sched, "one stream per image, %d band%s back to back", g.nbands, g.nbands == 1 ? "" : "s");
  if (split) {
    const int helpers = (nw == kSplitHalfWaves ? split_helpers<kModeSliced, kSplitHalfWaves>() : g.stage_x ? split_helpers<kModeSliced, kSplitWaves, true>() : split_helpers<kModeSliced, kSplitWaves, false>());
    char extra[48] = "";
    if (helpers) snprintf(extra, sizeof extra, " and %d that stage", helpers);
    snprintf(text, cap, "%s: %s, %lld workgroups of %d waves%s, %d channels each, 4 states per lane",
             fwd ? "m2d_fwd_split_kernel" : "m2d_bwd_split_kernel", sched, wgs, nw, extra, nw);
  }
  else {
    // (workgroups of 4 waves have waves that only stage, except in the backward that replays the forward between snapshots)
    const bool helped = !g.stacked && nw == kFwdHalfWaves && per_lane == 1 && (fwd || g.ck_shift == 0);
    char extra[48] = "";
    if (helped) snprintf(extra, sizeof extra, " and %d that stage", kWholeHelpers);
    snprintf(text, cap, "%s: %s, %lld workgroups of %d waves%s, %d channels each, 16 states per lane%s",
             fwd ? "m2d_fwd_kernel" : (g.ck_half ? "m2d_bwd2_kernel" : "m2d_bwd_kernel"), sched, wgs, nw, extra, nw * g.CS * per_lane,
             g.ck_half ? (fwd ? ", a snapshot every 2 steps" : ", a snapshot every 2 steps and one step in two recomputed") : "");
  }
  if (g.ck_shift) {
    const size_t n = strlen(text);
    if (n + 1 < cap) snprintf(text + n, cap - n, fwd ? ", a snapshot every %d steps" : ", a snapshot every %d steps and the forward replayed in between", kCK << g.ck_shift);
  }
  return M2D_OK;
}

int m2d_scan_link_error(const m2d_desc* desc, const void* workspace, void* stream, int* gave_up) {
  int rc = check_desc(desc);
  if (rc) return rc;
  if (!workspace || !gave_up) return M2D_ERR_NULL_POINTER;
  const Geometry g = make_geometry(desc);
  *gave_up = 0;
  if (!g.sliced) return M2D_OK;   // no workgroup of this problem waits for another
  hipStream_t st = static_cast<hipStream_t>(stream);
  uint32_t word = 0;
  if (hipStreamSynchronize(st) != hipSuccess) return M2D_ERR_HIP;
  if (hipMemcpy(&word, static_cast<const char*>(workspace) + g.prep_bytes, sizeof(word), hipMemcpyDeviceToHost) != hipSuccess) return M2D_ERR_HIP;
  *gave_up = word != 0;
  return M2D_OK;
}

int m2d_valu_rate_probe(int kind, int waves_per_simd, void* scratch, size_t scratch_bytes, void* stream, double* per_second) {
  if (!scratch || !per_second) return M2D_ERR_NULL_POINTER;
  if (kind < M2D_RATE_FMA || kind > M2D_RATE_SCAN_FWD_UNIT || waves_per_simd < 1 || waves_per_simd > 8) return M2D_ERR_UNSUPPORTED;
  const int cus = device_cus();
  const int blocks = cus * waves_per_simd;                 // 4 waves each: one per SIMD of a compute unit
  if (scratch_bytes < (size_t)blocks * 256 * sizeof(float)) return M2D_ERR_WORKSPACE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  float* out = static_cast<float*>(scratch);
  auto launch = [&] {
    switch (kind) {
      case M2D_RATE_FMA: hipLaunchKernelGGL(m2d_rate_probe_kernel<M2D_RATE_FMA>, dim3(blocks), dim3(256), 0, st, out, 1.0001f, 0.5f); break;
      case M2D_RATE_FMA_DEPENDENT: hipLaunchKernelGGL(m2d_rate_probe_kernel<M2D_RATE_FMA_DEPENDENT>, dim3(blocks), dim3(256), 0, st, out, 1.0001f, 0.5f); break;
      case M2D_RATE_EXP: hipLaunchKernelGGL(m2d_rate_probe_kernel<M2D_RATE_EXP>, dim3(blocks), dim3(256), 0, st, out, 1.0001f, 0.5f); break;
      case M2D_RATE_EXP_DEPENDENT: hipLaunchKernelGGL(m2d_rate_probe_kernel<M2D_RATE_EXP_DEPENDENT>, dim3(blocks), dim3(256), 0, st, out, 1.0001f, 0.5f); break;
      default: hipLaunchKernelGGL(m2d_rate_probe_kernel<M2D_RATE_SCAN_FWD_UNIT>, dim3(blocks), dim3(256), 0, st, out, 1.0001f, 0.5f); break;
    }
  };
  hipEvent_t e0 = nullptr, e1 = nullptr;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) { if (e0) (void)hipEventDestroy(e0); return M2D_ERR_HIP; }
  constexpr int kReps = 5;
  launch();   // (warm-up: code upload, clocks)
  (void)hipEventRecord(e0, st);
  for (int i = 0; i < kReps; ++i) launch();
  (void)hipEventRecord(e1, st);
  float ms = 0.f;
  const bool ok = hipGetLastError() == hipSuccess && hipEventSynchronize(e1) == hipSuccess && hipEventElapsedTime(&ms, e0, e1) == hipSuccess && ms > 0.f;
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (!ok) return M2D_ERR_HIP;
  // lane-operations (FMA, EXP kinds) or (cell, channel, state) units (the scan mix) per second, whole device
  *per_second = (double)blocks * 256 * 16.0 * kProbeIters * kReps / (ms * 1e-3);
  return M2D_OK;
}

int m2d_scan_fwd_noalloc(const m2d_desc* desc, const void* x, const void* deltaT, const void* deltaL, const void* AT,
                         const void* AL, const void* BT, const void* BL, const void* C, const void* D, void* y,
                         void* stream) {
  int rc = check_desc(desc);
  if (rc) return rc;
  if (workspace_bytes_of(make_geometry(desc), M2D_PASS_FWD, 0) > (size_t)M2D_NOALLOC_SCRATCH_BYTES) return M2D_ERR_TOO_LARGE;
  // address of the current device's copy of the array, looked up once per device
  static std::atomic<void*> addr[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return M2D_ERR_HIP;
  void* ws = addr[dev].load(std::memory_order_acquire);
  if (!ws) {
    if (hipGetSymbolAddress(&ws, HIP_SYMBOL(scratch)) != hipSuccess || !ws) return M2D_ERR_HIP;
    addr[dev].store(ws, std::memory_order_release);
  }
  // nothing in the workspace has to be zero on entry: the set-up kernel rewrites the page of zeros,
  // boundary rows and carried state are written before they are read
  return m2d_scan_fwd(desc, x, deltaT, deltaL, AT, AL, BT, BL, C, D, y, nullptr, 0, ws, (size_t)M2D_NOALLOC_SCRATCH_BYTES, stream);
}

}  // extern "C"

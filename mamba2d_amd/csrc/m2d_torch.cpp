// PyTorch-ROCm shim over the C ABI of libm2dscan.so (include/m2dscan.h).
//
// Registers two functional operators, m2dscan::scan_fwd and m2dscan::scan_bwd, which take the
// place of the reference's pair of in-place custom ops mamba2d::wf_fwd / mamba2d::wf_bwd
// (models/kernels/wavefront_cuda.py:25-57) plus the tensor algebra around them, and
// m2dscan::proj_fwd / m2dscan::proj_bwd for the projections that feed the scan
// (wavefront_cuda.py:63-95 and their autograd backward), and m2dscan::layernorm_fwd /
// m2dscan::dwconv3x3_fwd / starrelu_fwd / scale_residual_fwd for operators of the residual block at inference.  The shim only
// validates tensors, allocates outputs / scratch through the caching allocator, picks the
// current HIP stream and forwards raw pointers; all arithmetic lives behind the C ABI.
#include <ATen/ATen.h>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>
#include <torch/library.h>

#include <tuple>
#include <vector>

#include "m2dscan.h"

namespace {

using at::Tensor;

m2d_desc describe(const Tensor& x, const Tensor& AT, bool flip, bool raw_params = false, bool packed_bc = false,
                  bool dpre = false, int64_t ckpt_interval = 0) {
  TORCH_CHECK(x.dim() == 4, "m2dscan: x must be (B,H,W,E), got ", x.sizes());
  TORCH_CHECK(AT.dim() == 2, "m2dscan: AT must be (E,N), got ", AT.sizes());
  m2d_desc d{};
  d.B = static_cast<int32_t>(x.size(0));
  d.H = static_cast<int32_t>(x.size(1));
  d.W = static_cast<int32_t>(x.size(2));
  d.E = static_cast<int32_t>(x.size(3));
  d.N = static_cast<int32_t>(AT.size(1));
  if (x.scalar_type() == at::kFloat) d.dtype = M2D_F32;
  else if (x.scalar_type() == at::kBFloat16) d.dtype = M2D_BF16;
  else TORCH_CHECK(false, "m2dscan: float32 and bfloat16 are supported, got ", x.scalar_type());
  d.flags = (flip ? M2D_FLAG_FLIP : 0) | (raw_params ? M2D_FLAG_RAW_PARAMS : 0) | (packed_bc ? M2D_FLAG_PACKED_BC : 0) |
            (dpre ? M2D_FLAG_DPRE : 0);
  // (-4: a snapshot every 4 steps, kept in fp32 also for bf16 tensors, M2D_FLAG_FP32_SNAPSHOTS)
  TORCH_CHECK(ckpt_interval == 0 || ckpt_interval == 2 || ckpt_interval == 4 || ckpt_interval == 8 || ckpt_interval == 16 || ckpt_interval == -4,
              "m2dscan: ckpt_interval must be 0, 2, 4, 8 or 16 (or -4: every 4 steps, in fp32), got ", ckpt_interval);
  if (ckpt_interval == -4) d.flags |= M2D_FLAG_FP32_SNAPSHOTS;
  d.ckpt_interval = static_cast<int32_t>(ckpt_interval == -4 ? 4 : ckpt_interval);
  return d;
}

void expect(const Tensor& t, const char* name, const Tensor& x, at::IntArrayRef shape) {
  TORCH_CHECK(t.device() == x.device(), "m2dscan: ", name, " is on ", t.device(), ", x on ", x.device());
  TORCH_CHECK(t.scalar_type() == x.scalar_type(), "m2dscan: ", name, " has dtype ", t.scalar_type(),
              ", x has ", x.scalar_type(), " (all tensors share one dtype)");
  TORCH_CHECK(t.sizes() == shape, "m2dscan: ", name, " has shape ", t.sizes(), ", expected ", shape);
  TORCH_CHECK(t.is_contiguous(), "m2dscan: ", name, " must be contiguous");
}

void expect_param(const Tensor& t, const char* name, const Tensor& x, at::IntArrayRef shape, bool raw) {
  if (!raw) return expect(t, name, x, shape);
  TORCH_CHECK(t.device() == x.device(), "m2dscan: ", name, " is on ", t.device(), ", x on ", x.device());
  TORCH_CHECK(t.scalar_type() == at::kFloat, "m2dscan: ", name, " must be float32 when raw parameters are passed, got ", t.scalar_type());
  TORCH_CHECK(t.sizes() == shape, "m2dscan: ", name, " has shape ", t.sizes(), ", expected ", shape);
  TORCH_CHECK(t.is_contiguous(), "m2dscan: ", name, " must be contiguous");
}

void expect_all(const m2d_desc& d, const Tensor& x, const Tensor& dT, const Tensor& dL, const Tensor& AT,
                const Tensor& AL, const Tensor& BT, const Tensor& BL, const Tensor& C, const Tensor& D) {
  const bool raw = (d.flags & M2D_FLAG_RAW_PARAMS) != 0;
  TORCH_CHECK(x.is_cuda(), "m2dscan: tensors must live on the GPU");
  TORCH_CHECK(x.is_contiguous(), "m2dscan: x must be contiguous");
  const int64_t B = d.B, H = d.H, W = d.W, E = d.E, N = d.N;
  expect(dT, "deltaT", x, {B, H, W, E});
  expect(dL, "deltaL", x, {B, H, W, E});
  expect_param(AT, raw ? "AT_log" : "AT", x, {E, N}, raw);
  expect_param(AL, raw ? "AL_log" : "AL", x, {E, N}, raw);
  if (d.flags & M2D_FLAG_PACKED_BC) {   // BT holds the records written by proj_fwd; BL and C are not read
    TORCH_CHECK(BT.device() == x.device() && BT.scalar_type() == at::kFloat && BT.is_contiguous() &&
                BT.sizes() == at::IntArrayRef({B, H, W, 3 * N}),
                "m2dscan: packed B/C must be the contiguous float32 (B,H,W,48) tensor returned by proj_fwd");
  } else {
    expect(BT, "BT", x, {B, H, W, N});
    expect(BL, "BL", x, {B, H, W, N});
    expect(C, "C", x, {B, H, W, N});
  }
  expect_param(D, "D", x, {E}, raw);
}

void check(int status) { TORCH_CHECK(status == M2D_OK, "m2dscan: ", m2d_status_str(status), " (status ", status, ")"); }

Tensor bytes(size_t n, const Tensor& like) {
  return at::empty({static_cast<int64_t>(n > 0 ? n : 1)}, like.options().dtype(at::kByte));
}

std::tuple<Tensor, Tensor> scan_fwd(const Tensor& x, const Tensor& dT, const Tensor& dL, const Tensor& AT,
                                    const Tensor& AL, const Tensor& BT, const Tensor& BL, const Tensor& C,
                                    const Tensor& D, bool save_ckpt, bool flip, bool raw_params, bool packed_bc,
                                    int64_t ckpt_interval) {
  const m2d_desc d = describe(x, AT, flip, raw_params, packed_bc, false, ckpt_interval);
  expect_all(d, x, dT, dL, AT, AL, BT, BL, C, D);
  check(m2d_desc_check(&d));
  c10::DeviceGuard guard(x.device());
  Tensor y = at::empty_like(x);
  Tensor ck = bytes(save_ckpt ? m2d_scan_ckpt_bytes(&d) : 0, x);
  Tensor ws = bytes(m2d_scan_workspace_bytes(&d, M2D_PASS_FWD, save_ckpt), x);
  hipStream_t st = c10::hip::getCurrentHIPStream(x.device().index()).stream();
  check(m2d_scan_fwd(&d, x.data_ptr(), dT.data_ptr(), dL.data_ptr(), AT.data_ptr(), AL.data_ptr(), BT.data_ptr(),
                     BL.data_ptr(), C.data_ptr(), D.data_ptr(), y.data_ptr(), save_ckpt ? ck.data_ptr() : nullptr,
                     save_ckpt ? static_cast<size_t>(ck.numel()) : 0, ws.data_ptr(), static_cast<size_t>(ws.numel()),
                     st));
  return {y, ck};
}

std::vector<Tensor> scan_bwd(const Tensor& x, const Tensor& dT, const Tensor& dL, const Tensor& AT, const Tensor& AL,
                             const Tensor& BT, const Tensor& BL, const Tensor& C, const Tensor& D, const Tensor& dy,
                             const Tensor& ckpt, bool flip, bool raw_params, bool packed_bc, bool dpre,
                             int64_t ckpt_interval, bool sum_parts) {
  m2d_desc d = describe(x, AT, flip, raw_params, packed_bc, dpre, ckpt_interval);
  if (sum_parts) d.flags |= M2D_FLAG_SUM_PARTS;   // d_BT comes back as the fp32 per-workgroup sums for proj_bwd(sum_parts = its first size)
  expect_all(d, x, dT, dL, AT, AL, BT, BL, C, D);
  expect(dy, "dy", x, x.sizes());
  check(m2d_desc_check(&d));
  const bool have = ckpt.numel() > 1;   // a 1-byte tensor stands for "no checkpoints"
  if (have) {
    TORCH_CHECK(ckpt.device() == x.device() && ckpt.scalar_type() == at::kByte && ckpt.is_contiguous(),
                "m2dscan: ckpt must be the byte tensor returned by scan_fwd");
  }
  c10::DeviceGuard guard(x.device());
  const std::vector<int64_t> bc_shape = {d.B, d.H, d.W, d.N};
  std::vector<Tensor> g = {at::empty_like(x),  at::empty_like(dT), at::empty_like(dL), at::empty_like(AT), at::empty_like(AL),
                           at::empty(bc_shape, x.options()), at::empty(bc_shape, x.options()), at::empty(bc_shape, x.options()),
                           at::empty_like(D)};
  if (sum_parts) {
    g[5] = at::empty({m2d_scan_sum_parts(&d), d.B, d.H, d.W, 3 * d.N}, x.options().dtype(at::kFloat));
    g[6] = at::empty({0}, x.options());
    g[7] = at::empty({0}, x.options());
  }
  Tensor ws = bytes(m2d_scan_workspace_bytes(&d, M2D_PASS_BWD, have), x);
  hipStream_t st = c10::hip::getCurrentHIPStream(x.device().index()).stream();
  check(m2d_scan_bwd(&d, x.data_ptr(), dT.data_ptr(), dL.data_ptr(), AT.data_ptr(), AL.data_ptr(), BT.data_ptr(),
                     BL.data_ptr(), C.data_ptr(), D.data_ptr(), dy.data_ptr(), have ? ckpt.data_ptr() : nullptr,
                     have ? static_cast<size_t>(ckpt.numel()) : 0, g[0].data_ptr(), g[1].data_ptr(), g[2].data_ptr(),
                     g[3].data_ptr(), g[4].data_ptr(), g[5].data_ptr(), g[6].data_ptr(), g[7].data_ptr(),
                     g[8].data_ptr(), ws.data_ptr(), static_cast<size_t>(ws.numel()), st));
  return g;
}

// ---- projections either side of the scan (reference: proj_params, wavefront_cuda.py:63-95)
void expect_weight(const Tensor& t, const char* name, const Tensor& x, at::IntArrayRef shape) {
  TORCH_CHECK(t.device() == x.device(), "m2dscan: ", name, " is on ", t.device(), ", x on ", x.device());
  TORCH_CHECK(t.scalar_type() == at::kFloat, "m2dscan: ", name, " must be float32, got ", t.scalar_type());
  TORCH_CHECK(t.sizes() == shape, "m2dscan: ", name, " has shape ", t.sizes(), ", expected ", shape);
  TORCH_CHECK(t.is_contiguous(), "m2dscan: ", name, " must be contiguous");
}

m2d_desc describe_proj(const Tensor& x, int64_t N, bool round_weights, bool packed_bc = false) {
  TORCH_CHECK(x.dim() == 4 && x.is_cuda() && x.is_contiguous(), "m2dscan: x must be a contiguous (B,H,W,E) tensor on the GPU");
  m2d_desc d{};
  d.B = static_cast<int32_t>(x.size(0));
  d.H = static_cast<int32_t>(x.size(1));
  d.W = static_cast<int32_t>(x.size(2));
  d.E = static_cast<int32_t>(x.size(3));
  d.N = static_cast<int32_t>(N);
  if (x.scalar_type() == at::kFloat) d.dtype = M2D_F32;
  else if (x.scalar_type() == at::kBFloat16) d.dtype = M2D_BF16;
  else TORCH_CHECK(false, "m2dscan: float32 and bfloat16 are supported, got ", x.scalar_type());
  d.flags = (round_weights ? M2D_FLAG_ROUND_WEIGHTS : 0) | (packed_bc ? M2D_FLAG_PACKED_BC : 0);
  return d;
}

std::vector<Tensor> proj_fwd(const Tensor& x, const Tensor& Wx, const Tensor& wT, const Tensor& bT, const Tensor& wL,
                             const Tensor& bL, int64_t N, bool round_weights, bool packed_bc) {
  const m2d_desc d = describe_proj(x, N, round_weights, packed_bc);
  TORCH_CHECK(wT.dim() == 2, "m2dscan: dt_projT_w must be (E, dt_rank)");
  const int64_t B = d.B, H = d.H, W = d.W, E = d.E, R = wT.size(1);
  expect_weight(Wx, "x_proj_w", x, {2 * R + 3 * N, E});
  expect_weight(wT, "dt_projT_w", x, {E, R});
  expect_weight(bT, "dt_projT_b", x, {E});
  expect_weight(wL, "dt_projL_w", x, {E, R});
  expect_weight(bL, "dt_projL_b", x, {E});
  c10::DeviceGuard guard(x.device());
  // packed: one float32 (B,H,W,48) tensor of records in the BT place, empty tensors for BL and C
  std::vector<Tensor> o = {at::empty({B, H, W, 2 * R}, x.options()), at::empty_like(x), at::empty_like(x),
                           packed_bc ? at::empty({B, H, W, 3 * N}, x.options().dtype(at::kFloat)) : at::empty({B, H, W, N}, x.options()),
                           packed_bc ? at::empty({0}, x.options()) : at::empty({B, H, W, N}, x.options()),
                           packed_bc ? at::empty({0}, x.options()) : at::empty({B, H, W, N}, x.options())};
  const size_t need = m2d_proj_workspace_bytes(&d, static_cast<int>(R), M2D_PASS_FWD);
  TORCH_CHECK(need > 0, "m2dscan: projection shapes outside what the kernels are built for (N = 16, dt_rank <= 32, E <= 4096)");
  Tensor ws = bytes(need, x);
  hipStream_t st = c10::hip::getCurrentHIPStream(x.device().index()).stream();
  check(m2d_proj_fwd(&d, static_cast<int>(R), x.data_ptr(), Wx.data_ptr<float>(), wT.data_ptr<float>(), bT.data_ptr<float>(),
                     wL.data_ptr<float>(), bL.data_ptr<float>(), o[0].data_ptr(), o[1].data_ptr(), o[2].data_ptr(),
                     o[3].data_ptr(), o[4].data_ptr(), o[5].data_ptr(), ws.data_ptr(), static_cast<size_t>(ws.numel()), st));
  return o;
}

// Returns a tuple, not a list: the operator writes into dx, and torch.compile can only functionalise a
// mutating custom operator whose results are plain tensors.
std::tuple<Tensor, Tensor, Tensor, Tensor, Tensor> proj_bwd(const Tensor& x, const Tensor& low, const Tensor& dT, const Tensor& dL, const Tensor& Wx,
                             const Tensor& wT, const Tensor& wL, const Tensor& ddT, const Tensor& ddL, const Tensor& dBT,
                             const Tensor& dBL, const Tensor& dC, Tensor dx, bool round_weights, bool dpre, int64_t sum_parts) {
  TORCH_CHECK(sum_parts >= 0 && dBT.dim() == (sum_parts ? 5 : 4) && wT.dim() == 2,
              "m2dscan: d_BT must be (B,H,W,N), or (sum_parts,B,H,W,3N) as scan_bwd(sum_parts=True) returns it, and dt_projT_w (E, dt_rank)");
  const int64_t N = sum_parts ? dBT.size(4) / 3 : dBT.size(3);
  m2d_desc d = describe_proj(x, N, round_weights);
  if (dpre) d.flags |= M2D_FLAG_DPRE;   // d_deltaT, d_deltaL are gradients before the softplus; deltaT, deltaL are not read
  const int64_t B = d.B, H = d.H, W = d.W, E = d.E, R = wT.size(1);
  expect_weight(Wx, "x_proj_w", x, {2 * R + 3 * N, E});
  expect_weight(wT, "dt_projT_w", x, {E, R});
  expect_weight(wL, "dt_projL_w", x, {E, R});
  expect(low, "lowrank", x, {B, H, W, 2 * R});
  expect(dT, "deltaT", x, {B, H, W, E});
  expect(dL, "deltaL", x, {B, H, W, E});
  expect(ddT, "d_deltaT", x, {B, H, W, E});
  expect(ddL, "d_deltaL", x, {B, H, W, E});
  if (sum_parts) {
    TORCH_CHECK(dBT.device() == x.device() && dBT.scalar_type() == at::kFloat && dBT.is_contiguous() &&
                dBT.sizes() == at::IntArrayRef({sum_parts, B, H, W, 3 * N}),
                "m2dscan: d_BT must be the contiguous float32 (sum_parts,B,H,W,3N) tensor of scan_bwd(sum_parts=True)");
  } else {
    expect(dBT, "d_BT", x, {B, H, W, N});
    expect(dBL, "d_BL", x, {B, H, W, N});
    expect(dC, "d_C", x, {B, H, W, N});
  }
  expect(dx, "dx", x, {B, H, W, E});
  c10::DeviceGuard guard(x.device());
  std::vector<Tensor> g = {at::empty_like(Wx), at::empty_like(wT), at::empty({E}, wT.options()), at::empty_like(wL),
                           at::empty({E}, wT.options())};
  const size_t need = m2d_proj_workspace_bytes(&d, static_cast<int>(R), M2D_PASS_BWD);
  TORCH_CHECK(need > 0, "m2dscan: projection shapes outside what the kernels are built for (N = 16, dt_rank <= 32, E <= 4096)");
  Tensor ws = bytes(need, x);
  hipStream_t st = c10::hip::getCurrentHIPStream(x.device().index()).stream();
  check(m2d_proj_bwd_parts(&d, static_cast<int>(R), static_cast<int>(sum_parts), x.data_ptr(), low.data_ptr(), dT.data_ptr(), dL.data_ptr(),
                     Wx.data_ptr<float>(), wT.data_ptr<float>(), wL.data_ptr<float>(), ddT.data_ptr(), ddL.data_ptr(),
                     dBT.data_ptr(), dBL.data_ptr(), dC.data_ptr(), dx.data_ptr(), g[0].data_ptr<float>(),
                     g[1].data_ptr<float>(), g[2].data_ptr<float>(), g[3].data_ptr<float>(), g[4].data_ptr<float>(),
                     ws.data_ptr(), static_cast<size_t>(ws.numel()), st));
  return std::make_tuple(g[0], g[1], g[2], g[3], g[4]);
}

// ---- operators of the residual block (inference forward)
int dtype_code(const Tensor& t, const char* name) {
  if (t.scalar_type() == at::kFloat) return M2D_F32;
  if (t.scalar_type() == at::kBFloat16) return M2D_BF16;
  TORCH_CHECK(false, "m2dscan: ", name, " must be float32 or bfloat16, got ", t.scalar_type());
  return 0;
}

Tensor layernorm_fwd(const Tensor& x, const Tensor& weight, const Tensor& bias, double eps) {
  TORCH_CHECK(x.is_cuda() && x.dim() >= 1 && x.is_contiguous(), "m2dscan: x must be a contiguous tensor on the GPU");
  const int64_t C = x.size(-1);
  TORCH_CHECK(weight.sizes() == at::IntArrayRef({C}) && bias.sizes() == at::IntArrayRef({C}) && weight.is_contiguous() &&
              bias.is_contiguous() && weight.device() == x.device() && bias.device() == x.device() &&
              weight.scalar_type() == bias.scalar_type(),
              "m2dscan: weight and bias must be contiguous (", C, ",) tensors of one dtype on x's device");
  c10::DeviceGuard guard(x.device());
  Tensor y = at::empty_like(x);
  if (x.numel() == 0) return y;
  hipStream_t st = c10::hip::getCurrentHIPStream(x.device().index()).stream();
  check(m2d_layernorm_fwd(x.numel() / C, static_cast<int>(C), dtype_code(x, "x"), dtype_code(weight, "weight"), x.data_ptr(),
                          weight.data_ptr(), bias.data_ptr(), static_cast<float>(eps), y.data_ptr(), st));
  return y;
}

Tensor dwconv3x3_fwd(const Tensor& x, const Tensor& weight) {
  TORCH_CHECK(x.is_cuda() && x.dim() == 4 && x.is_contiguous(), "m2dscan: x must be a contiguous (B,H,W,C) tensor on the GPU");
  const int64_t C = x.size(3);
  TORCH_CHECK(weight.sizes() == at::IntArrayRef({C, 1, 3, 3}) && weight.is_contiguous() && weight.device() == x.device(),
              "m2dscan: weight must be a contiguous (", C, ",1,3,3) tensor on x's device");
  c10::DeviceGuard guard(x.device());
  Tensor y = at::empty_like(x);
  if (x.numel() == 0) return y;
  hipStream_t st = c10::hip::getCurrentHIPStream(x.device().index()).stream();
  check(m2d_dwconv3x3_fwd(static_cast<int>(x.size(0)), static_cast<int>(x.size(1)), static_cast<int>(x.size(2)),
                          static_cast<int>(C), dtype_code(x, "x"), dtype_code(weight, "weight"), x.data_ptr(), weight.data_ptr(),
                          y.data_ptr(), st));
  return y;
}

Tensor starrelu_fwd(const Tensor& x, const Tensor& scale, const Tensor& bias) {
  TORCH_CHECK(x.is_cuda() && x.is_contiguous(), "m2dscan: x must be a contiguous tensor on the GPU");
  TORCH_CHECK(scale.numel() == 1 && bias.numel() == 1 && scale.device() == x.device() && bias.device() == x.device() &&
              scale.scalar_type() == bias.scalar_type(), "m2dscan: scale and bias must hold one element each, of one dtype, on x's device");
  c10::DeviceGuard guard(x.device());
  Tensor y = at::empty_like(x);
  if (x.numel() == 0) return y;
  hipStream_t st = c10::hip::getCurrentHIPStream(x.device().index()).stream();
  check(m2d_starrelu_fwd(x.numel(), dtype_code(x, "x"), dtype_code(scale, "scale"), x.data_ptr(), scale.data_ptr(), bias.data_ptr(),
                         y.data_ptr(), st));
  return y;
}

Tensor scale_residual_fwd(const Tensor& x, const Tensor& scale, const Tensor& residual, const c10::optional<Tensor>& residual2) {
  TORCH_CHECK(x.is_cuda() && x.dim() >= 1 && x.is_contiguous(), "m2dscan: x must be a contiguous tensor on the GPU");
  for (const Tensor* r : {&residual, residual2.has_value() ? &*residual2 : &residual})
    TORCH_CHECK(r->is_contiguous() && r->sizes() == x.sizes() && r->scalar_type() == x.scalar_type() && r->device() == x.device(),
                "m2dscan: x and the residuals must be contiguous tensors of one shape and dtype on the GPU");
  const int64_t C = x.size(-1);
  TORCH_CHECK(scale.sizes() == at::IntArrayRef({C}) && scale.is_contiguous() && scale.device() == x.device(),
              "m2dscan: scale must be a contiguous (", C, ",) tensor on x's device");
  c10::DeviceGuard guard(x.device());
  Tensor y = at::empty_like(x);
  if (x.numel() == 0) return y;
  hipStream_t st = c10::hip::getCurrentHIPStream(x.device().index()).stream();
  check(m2d_scale_residual_fwd(x.numel() / C, static_cast<int>(C), dtype_code(x, "x"), dtype_code(scale, "scale"), x.data_ptr(),
                               scale.data_ptr(), residual.data_ptr(), residual2.has_value() ? residual2->data_ptr() : nullptr,
                               y.data_ptr(), st));
  return y;
}

std::tuple<Tensor, Tensor> scale_residual_layernorm_fwd(const Tensor& x, const Tensor& scale, const Tensor& residual,
                                                        const c10::optional<Tensor>& residual2, const Tensor& weight,
                                                        const Tensor& bias, double eps) {
  TORCH_CHECK(x.is_cuda() && x.dim() >= 1 && x.is_contiguous(), "m2dscan: x must be a contiguous tensor on the GPU");
  for (const Tensor* r : {&residual, residual2.has_value() ? &*residual2 : &residual})
    TORCH_CHECK(r->is_contiguous() && r->sizes() == x.sizes() && r->scalar_type() == x.scalar_type() && r->device() == x.device(),
                "m2dscan: x and the residuals must be contiguous tensors of one shape and dtype on the GPU");
  const int64_t C = x.size(-1);
  for (const Tensor* t : {&scale, &weight, &bias})
    TORCH_CHECK(t->sizes() == at::IntArrayRef({C}) && t->is_contiguous() && t->device() == x.device() &&
                t->scalar_type() == scale.scalar_type(), "m2dscan: scale, weight and bias must be contiguous (", C,
                ",) tensors of one dtype on x's device");
  c10::DeviceGuard guard(x.device());
  Tensor xo = at::empty_like(x), y = at::empty_like(x);
  if (x.numel() == 0) return {xo, y};
  hipStream_t st = c10::hip::getCurrentHIPStream(x.device().index()).stream();
  check(m2d_scale_residual_layernorm_fwd(x.numel() / C, static_cast<int>(C), dtype_code(x, "x"), dtype_code(scale, "scale"),
                                         x.data_ptr(), scale.data_ptr(), residual.data_ptr(),
                                         residual2.has_value() ? residual2->data_ptr() : nullptr, weight.data_ptr(),
                                         bias.data_ptr(), static_cast<float>(eps), xo.data_ptr(), y.data_ptr(), st));
  return {xo, y};
}

std::tuple<Tensor, Tensor> rope_qknorm_fwd(const Tensor& qkv, const Tensor& cos, const Tensor& sin, const Tensor& qw,
                                           const Tensor& qb, const Tensor& kw, const Tensor& kb, double eps, bool token_major) {
  TORCH_CHECK(qkv.is_cuda() && qkv.dim() == 5 && qkv.size(2) == 3 && qkv.is_contiguous(),
              "m2dscan: qkv must be a contiguous (B, L, 3, heads, head_dim) tensor on the GPU");
  const int64_t B = qkv.size(0), L = qkv.size(1), nh = qkv.size(3), hd = qkv.size(4);
  for (const Tensor* t : {&cos, &sin})
    TORCH_CHECK(t->sizes() == at::IntArrayRef({L, hd}) && t->scalar_type() == qkv.scalar_type() && t->device() == qkv.device() &&
                t->is_contiguous(), "m2dscan: cos and sin must be contiguous (", L, ",", hd, ") tensors of qkv's dtype and device");
  for (const Tensor* t : {&qw, &qb, &kw, &kb})
    TORCH_CHECK(t->sizes() == at::IntArrayRef({hd}) && t->scalar_type() == qw.scalar_type() && t->device() == qkv.device() &&
                t->is_contiguous(), "m2dscan: the LayerNorm weights must be contiguous (", hd, ",) tensors of one dtype on qkv's device");
  c10::DeviceGuard guard(qkv.device());
  // (B, heads, L, hd) tensors either way; token-major they are views of (B, L, heads, hd) memory
  Tensor q = token_major ? at::empty({B, L, nh, hd}, qkv.options()).permute({0, 2, 1, 3}) : at::empty({B, nh, L, hd}, qkv.options());
  Tensor k = token_major ? at::empty({B, L, nh, hd}, qkv.options()).permute({0, 2, 1, 3}) : at::empty({B, nh, L, hd}, qkv.options());
  if (qkv.numel() == 0) return {q, k};
  hipStream_t st = c10::hip::getCurrentHIPStream(qkv.device().index()).stream();
  check(m2d_rope_qknorm_fwd(static_cast<int>(B), static_cast<int>(L), static_cast<int>(nh), static_cast<int>(hd),
                            dtype_code(qkv, "qkv"), dtype_code(qw, "q_weight"), qkv.data_ptr(), cos.data_ptr(), sin.data_ptr(),
                            qw.data_ptr(), qb.data_ptr(), kw.data_ptr(), kb.data_ptr(), static_cast<float>(eps), token_major ? 1 : 0,
                            q.data_ptr(), k.data_ptr(), st));
  return {q, k};
}

Tensor mlp_fwd(const Tensor& x, const Tensor& w1, const c10::optional<Tensor>& b1, const Tensor& w2,
               const c10::optional<Tensor>& b2, const c10::optional<Tensor>& ln_weight, const c10::optional<Tensor>& ln_bias,
               double eps) {
  TORCH_CHECK(x.is_cuda() && x.dim() >= 1 && x.is_contiguous() && x.scalar_type() == at::kBFloat16,
              "m2dscan: x must be a contiguous bfloat16 tensor on the GPU");
  const int64_t C = x.size(-1);
  TORCH_CHECK(w1.dim() == 2 && w1.size(1) == C && w1.is_contiguous() && w1.device() == x.device(),
              "m2dscan: w1 must be a contiguous (hidden,", C, ") tensor on x's device");
  const int64_t H = w1.size(0);
  TORCH_CHECK(w2.sizes() == at::IntArrayRef({C, H}) && w2.is_contiguous() && w2.device() == x.device() &&
              w2.scalar_type() == w1.scalar_type(), "m2dscan: w2 must be a contiguous (", C, ",", H, ") tensor of w1's dtype and device");
  auto small = [&](const c10::optional<Tensor>& t, int64_t n, const char* name) -> const void* {
    if (!t.has_value() || !t->defined()) return nullptr;
    TORCH_CHECK(t->numel() == n && t->is_contiguous() && t->device() == x.device() && t->scalar_type() == w1.scalar_type(),
                "m2dscan: ", name, " must hold ", n, " elements of the weights' dtype on x's device");
    return t->data_ptr();
  };
  const void* b1p = small(b1, H, "b1");
  const void* b2p = small(b2, C, "b2");
  const void* lw = small(ln_weight, C, "ln_weight");
  const void* lb = small(ln_bias, C, "ln_bias");
  TORCH_CHECK((lw != nullptr) == (lb != nullptr), "m2dscan: ln_weight and ln_bias come together");
  c10::DeviceGuard guard(x.device());
  Tensor y = at::empty_like(x);
  if (x.numel() == 0) return y;
  hipStream_t st = c10::hip::getCurrentHIPStream(x.device().index()).stream();
  check(m2d_mlp_fwd(x.numel() / C, static_cast<int>(C), static_cast<int>(H), dtype_code(w1, "w1"), x.data_ptr(), lw, lb,
                    static_cast<float>(eps), w1.data_ptr(), b1p, w2.data_ptr(), b2p, y.data_ptr(), st));
  return y;
}

Tensor rope_attention_fwd(const Tensor& qkv, const Tensor& cos, const Tensor& sin, const Tensor& qw, const Tensor& qb,
                          const Tensor& kw, const Tensor& kb, double eps, double scale) {
  TORCH_CHECK(qkv.is_cuda() && qkv.dim() == 5 && qkv.size(2) == 3 && qkv.is_contiguous() && qkv.scalar_type() == at::kBFloat16,
              "m2dscan: qkv must be a contiguous bfloat16 (B, L, 3, heads, head_dim) tensor on the GPU");
  const int64_t B = qkv.size(0), L = qkv.size(1), nh = qkv.size(3), hd = qkv.size(4);
  for (const Tensor* t : {&cos, &sin})
    TORCH_CHECK(t->sizes() == at::IntArrayRef({L, hd}) && t->scalar_type() == qkv.scalar_type() && t->device() == qkv.device() &&
                t->is_contiguous(), "m2dscan: cos and sin must be contiguous (", L, ",", hd, ") tensors of qkv's dtype and device");
  for (const Tensor* t : {&qw, &qb, &kw, &kb})
    TORCH_CHECK(t->sizes() == at::IntArrayRef({hd}) && t->scalar_type() == qw.scalar_type() && t->device() == qkv.device() &&
                t->is_contiguous(), "m2dscan: the LayerNorm weights must be contiguous (", hd, ",) tensors of one dtype on qkv's device");
  c10::DeviceGuard guard(qkv.device());
  Tensor out = at::empty({B, L, nh, hd}, qkv.options());
  if (qkv.numel() == 0) return out;
  hipStream_t st = c10::hip::getCurrentHIPStream(qkv.device().index()).stream();
  check(m2d_rope_attention_fwd(static_cast<int>(B), static_cast<int>(L), static_cast<int>(nh), static_cast<int>(hd),
                               dtype_code(qw, "q_weight"), qkv.data_ptr(), cos.data_ptr(), sin.data_ptr(), qw.data_ptr(),
                               qb.data_ptr(), kw.data_ptr(), kb.data_ptr(), static_cast<float>(eps), static_cast<float>(scale),
                               out.data_ptr(), st));
  return out;
}

Tensor linear_act_fwd(const Tensor& x, const Tensor& weight, const c10::optional<Tensor>& bias, int64_t pre,
                      const c10::optional<Tensor>& pre_scale, const c10::optional<Tensor>& pre_bias, int64_t post,
                      const c10::optional<Tensor>& post_scale, const c10::optional<Tensor>& post_bias) {
  TORCH_CHECK(x.is_cuda() && x.dim() >= 1 && x.is_contiguous() && x.scalar_type() == at::kBFloat16,
              "m2dscan: x must be a contiguous bfloat16 tensor on the GPU");
  const int64_t K = x.size(-1);
  TORCH_CHECK(weight.dim() == 2 && weight.size(1) == K && weight.is_contiguous() && weight.device() == x.device(),
              "m2dscan: weight must be a contiguous (N,", K, ") tensor on x's device");
  const int64_t N = weight.size(0);
  auto small = [&](const c10::optional<Tensor>& t, int64_t n, const char* name) -> const void* {
    if (!t.has_value() || !t->defined()) return nullptr;
    TORCH_CHECK(t->numel() == n && t->is_contiguous() && t->device() == x.device() && t->scalar_type() == weight.scalar_type(),
                "m2dscan: ", name, " must hold ", n, " elements of the weight's dtype on x's device");
    return t->data_ptr();
  };
  const void* b = small(bias, N, "bias");
  const void* ps = small(pre_scale, 1, "pre_scale");
  const void* pb = small(pre_bias, 1, "pre_bias");
  const void* qs = small(post_scale, 1, "post_scale");
  const void* qb = small(post_bias, 1, "post_bias");
  c10::DeviceGuard guard(x.device());
  std::vector<int64_t> shape(x.sizes().begin(), x.sizes().end());
  shape.back() = N;
  Tensor y = at::empty(shape, x.options());
  if (x.numel() == 0) return y;
  hipStream_t st = c10::hip::getCurrentHIPStream(x.device().index()).stream();
  check(m2d_linear_fwd(x.numel() / K, static_cast<int>(K), static_cast<int>(N), dtype_code(weight, "weight"), x.data_ptr(),
                       weight.data_ptr(), b, static_cast<int>(pre), ps, pb, static_cast<int>(post), qs, qb, y.data_ptr(), st));
  return y;
}

Tensor layernorm_linear_act_fwd(const Tensor& x, const Tensor& ln_weight, const Tensor& ln_bias, double eps, const Tensor& weight,
                                const c10::optional<Tensor>& bias, int64_t post, const c10::optional<Tensor>& post_scale,
                                const c10::optional<Tensor>& post_bias) {
  TORCH_CHECK(x.is_cuda() && x.dim() >= 1 && x.is_contiguous() && x.scalar_type() == at::kBFloat16,
              "m2dscan: x must be a contiguous bfloat16 tensor on the GPU");
  const int64_t K = x.size(-1);
  TORCH_CHECK(weight.dim() == 2 && weight.size(1) == K && weight.is_contiguous() && weight.device() == x.device(),
              "m2dscan: weight must be a contiguous (N,", K, ") tensor on x's device");
  const int64_t N = weight.size(0);
  auto small = [&](const c10::optional<Tensor>& t, int64_t n, const char* name) -> const void* {
    if (!t.has_value() || !t->defined()) return nullptr;
    TORCH_CHECK(t->numel() == n && t->is_contiguous() && t->device() == x.device() && t->scalar_type() == weight.scalar_type(),
                "m2dscan: ", name, " must hold ", n, " elements of the weight's dtype on x's device");
    return t->data_ptr();
  };
  const void* lw = small(ln_weight, K, "ln_weight");
  const void* lb = small(ln_bias, K, "ln_bias");
  const void* b = small(bias, N, "bias");
  const void* qs = small(post_scale, 1, "post_scale");
  const void* qb = small(post_bias, 1, "post_bias");
  c10::DeviceGuard guard(x.device());
  std::vector<int64_t> shape(x.sizes().begin(), x.sizes().end());
  shape.back() = N;
  Tensor y = at::empty(shape, x.options());
  if (x.numel() == 0) return y;
  hipStream_t st = c10::hip::getCurrentHIPStream(x.device().index()).stream();
  check(m2d_layernorm_linear_fwd(x.numel() / K, static_cast<int>(K), static_cast<int>(N), dtype_code(weight, "weight"), x.data_ptr(),
                                 lw, lb, static_cast<float>(eps), weight.data_ptr(), b, static_cast<int>(post), qs, qb, y.data_ptr(), st));
  return y;
}

int64_t abi_version() { return m2d_version(); }

// ---- the reference's own pair of in-place operators, mamba2d::wf_fwd and mamba2d::wf_bwd (wavefront_cuda.py:25-57),
// for callers that use them directly: same names, argument order and mutated arguments; any number of states;
// float64, float32 and bfloat16 (wf_cuda.cu:182,240).  They materialise hs and are not on the fast path.
int wf_dtype(const Tensor& hs) {
  if (hs.scalar_type() == at::kFloat) return M2D_F32;
  if (hs.scalar_type() == at::kBFloat16) return M2D_BF16;
  if (hs.scalar_type() == at::kDouble) return M2D_F64;
  TORCH_CHECK(false, "mamba2d::wf_*: float64, float32 and bfloat16 are supported, got ", hs.scalar_type());
}
void wf_expect(const Tensor& t, const char* name, const Tensor& hs, at::IntArrayRef shape) {
  TORCH_CHECK(t.device() == hs.device(), "mamba2d::wf_*: ", name, " is on ", t.device(), ", hs on ", hs.device());
  TORCH_CHECK(t.scalar_type() == hs.scalar_type(), "mamba2d::wf_*: ", name, " has dtype ", t.scalar_type(), ", hs has ",
              hs.scalar_type(), " (all tensors share one dtype, as the reference's accessors require)");
  TORCH_CHECK(t.sizes() == shape, "mamba2d::wf_*: ", name, " has shape ", t.sizes(), ", expected ", shape);
  TORCH_CHECK(t.is_contiguous(), "mamba2d::wf_*: ", name, " must be contiguous");
}

void wf_fwd(Tensor& hs, const Tensor& x, const Tensor& dT, const Tensor& dL, const Tensor& BT, const Tensor& BL,
            const Tensor& AT, const Tensor& AL) {
  TORCH_CHECK(hs.dim() == 5 && hs.is_contiguous(), "mamba2d::wf_fwd: hs must be a contiguous (B,H,W,E,N) tensor, got ", hs.sizes());
  const int64_t B = hs.size(0), H = hs.size(1), W = hs.size(2), E = hs.size(3), N = hs.size(4);
  wf_expect(x, "x", hs, {B, H, W, E}); wf_expect(dT, "deltaT", hs, {B, H, W, E}); wf_expect(dL, "deltaL", hs, {B, H, W, E});
  wf_expect(BT, "BT", hs, {B, H, W, N}); wf_expect(BL, "BL", hs, {B, H, W, N});
  wf_expect(AT, "AT", hs, {E, N}); wf_expect(AL, "AL", hs, {E, N});
  c10::DeviceGuard guard(hs.device());
  hipStream_t st = c10::hip::getCurrentHIPStream(hs.device().index()).stream();
  check(m2d_wf_fwd((int)B, (int)H, (int)W, (int)E, (int)N, wf_dtype(hs), hs.data_ptr(), x.data_ptr(), dT.data_ptr(), dL.data_ptr(),
                   BT.data_ptr(), BL.data_ptr(), AT.data_ptr(), AL.data_ptr(), st));
}

void wf_bwd(const Tensor& hs, const Tensor& x, const Tensor& dT, const Tensor& dL, const Tensor& AT, const Tensor& AL,
            Tensor& grad_output, Tensor& dDAT, Tensor& dDAL, Tensor& omega) {
  TORCH_CHECK(hs.dim() == 5 && hs.is_contiguous(), "mamba2d::wf_bwd: hs must be a contiguous (B,H,W,E,N) tensor, got ", hs.sizes());
  const int64_t B = hs.size(0), H = hs.size(1), W = hs.size(2), E = hs.size(3), N = hs.size(4);
  wf_expect(x, "x", hs, {B, H, W, E}); wf_expect(dT, "deltaT", hs, {B, H, W, E}); wf_expect(dL, "deltaL", hs, {B, H, W, E});
  wf_expect(AT, "AT", hs, {E, N}); wf_expect(AL, "AL", hs, {E, N});
  wf_expect(grad_output, "grad_output", hs, hs.sizes()); wf_expect(dDAT, "dDAT", hs, hs.sizes()); wf_expect(dDAL, "dDAL", hs, hs.sizes());
  wf_expect(omega, "omega", hs, {2, B, H, E, N});
  c10::DeviceGuard guard(hs.device());
  hipStream_t st = c10::hip::getCurrentHIPStream(hs.device().index()).stream();
  check(m2d_wf_bwd((int)B, (int)H, (int)W, (int)E, (int)N, wf_dtype(hs), hs.data_ptr(), x.data_ptr(), dT.data_ptr(), dL.data_ptr(),
                   AT.data_ptr(), AL.data_ptr(), grad_output.data_ptr(), dDAT.data_ptr(), dDAL.data_ptr(), omega.data_ptr(), st));
}


}  // namespace

TORCH_LIBRARY(m2dscan, m) {
  m.def("scan_fwd(Tensor x, Tensor deltaT, Tensor deltaL, Tensor AT, Tensor AL, Tensor BT, Tensor BL, Tensor C, "
        "Tensor D, bool save_ckpt, bool flip, bool raw_params=False, bool packed_bc=False, int ckpt_interval=0) -> (Tensor, Tensor)");
  m.def("scan_bwd(Tensor x, Tensor deltaT, Tensor deltaL, Tensor AT, Tensor AL, Tensor BT, Tensor BL, Tensor C, "
        "Tensor D, Tensor dy, Tensor ckpt, bool flip, bool raw_params=False, bool packed_bc=False, bool dpre=False, "
        "int ckpt_interval=0, bool sum_parts=False) -> Tensor[]");
  m.def("proj_fwd(Tensor x, Tensor x_proj_w, Tensor dt_projT_w, Tensor dt_projT_b, Tensor dt_projL_w, Tensor dt_projL_b, "
        "int d_state, bool round_weights, bool packed_bc=False) -> Tensor[]");
  m.def("proj_bwd(Tensor x, Tensor lowrank, Tensor deltaT, Tensor deltaL, Tensor x_proj_w, Tensor dt_projT_w, "
        "Tensor dt_projL_w, Tensor d_deltaT, Tensor d_deltaL, Tensor d_BT, Tensor d_BL, Tensor d_C, Tensor(a!) dx, "
        "bool round_weights, bool dpre=False, int sum_parts=0) -> (Tensor, Tensor, Tensor, Tensor, Tensor)");
  m.def("layernorm_fwd(Tensor x, Tensor weight, Tensor bias, float eps) -> Tensor");
  m.def("dwconv3x3_fwd(Tensor x, Tensor weight) -> Tensor");
  m.def("starrelu_fwd(Tensor x, Tensor scale, Tensor bias) -> Tensor");
  m.def("scale_residual_fwd(Tensor x, Tensor scale, Tensor residual, Tensor? residual2=None) -> Tensor");
  m.def("scale_residual_layernorm_fwd(Tensor x, Tensor scale, Tensor residual, Tensor? residual2, Tensor weight, Tensor bias, "
        "float eps) -> (Tensor, Tensor)");
  m.def("rope_qknorm_fwd(Tensor qkv, Tensor cos, Tensor sin, Tensor q_weight, Tensor q_bias, Tensor k_weight, Tensor k_bias, "
        "float eps, bool token_major=False) -> (Tensor, Tensor)");
  m.def("mlp_fwd(Tensor x, Tensor w1, Tensor? b1, Tensor w2, Tensor? b2, Tensor? ln_weight=None, Tensor? ln_bias=None, "
        "float eps=1e-5) -> Tensor");
  m.def("layernorm_linear_act_fwd(Tensor x, Tensor ln_weight, Tensor ln_bias, float eps, Tensor weight, Tensor? bias, int post, "
        "Tensor? post_scale, Tensor? post_bias) -> Tensor");
  m.def("rope_attention_fwd(Tensor qkv, Tensor cos, Tensor sin, Tensor q_weight, Tensor q_bias, Tensor k_weight, Tensor k_bias, "
        "float eps, float scale) -> Tensor");
  m.def("linear_act_fwd(Tensor x, Tensor weight, Tensor? bias, int pre, Tensor? pre_scale, Tensor? pre_bias, int post, "
        "Tensor? post_scale, Tensor? post_bias) -> Tensor");
  m.def("abi_version() -> int", &abi_version);
}

TORCH_LIBRARY_IMPL(m2dscan, CUDA, m) {   // ROCm devices dispatch under the CUDA key
  m.impl("scan_fwd", &scan_fwd);
  m.impl("scan_bwd", &scan_bwd);
  m.impl("proj_fwd", &proj_fwd);
  m.impl("proj_bwd", &proj_bwd);
  m.impl("layernorm_fwd", &layernorm_fwd);
  m.impl("dwconv3x3_fwd", &dwconv3x3_fwd);
  m.impl("starrelu_fwd", &starrelu_fwd);
  m.impl("scale_residual_fwd", &scale_residual_fwd);
  m.impl("rope_qknorm_fwd", &rope_qknorm_fwd);
  m.impl("scale_residual_layernorm_fwd", &scale_residual_layernorm_fwd);
  m.impl("rope_attention_fwd", &rope_attention_fwd);
  m.impl("mlp_fwd", &mlp_fwd);
  m.impl("layernorm_linear_act_fwd", &layernorm_linear_act_fwd);
  m.impl("linear_act_fwd", &linear_act_fwd);
}

TORCH_LIBRARY(mamba2d, m) {   // the reference's operator names (wavefront_cuda.py:25, :40), same mutated arguments
  m.def("wf_fwd(Tensor(a!) hs, Tensor x, Tensor deltaT, Tensor deltaL, Tensor BT, Tensor BL, Tensor AT, Tensor AL) -> ()");
  m.def("wf_bwd(Tensor hs, Tensor x, Tensor deltaT, Tensor deltaL, Tensor AT, Tensor AL, Tensor(a!) grad_output, "
        "Tensor(b!) dDAT, Tensor(c!) dDAL, Tensor(d!) omega) -> ()");
}

TORCH_LIBRARY_IMPL(mamba2d, CUDA, m) {
  m.impl("wf_fwd", &wf_fwd);
  m.impl("wf_bwd", &wf_bwd);
}

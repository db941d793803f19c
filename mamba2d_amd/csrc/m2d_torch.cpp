// PyTorch-ROCm shim over the C ABI of libm2dscan.so (include/m2dscan.h).
//
// Registers two functional operators, m2dscan::scan_fwd and m2dscan::scan_bwd, which take the
// place of the reference's pair of in-place custom ops mamba2d::wf_fwd / mamba2d::wf_bwd
// (models/kernels/wavefront_cuda.py:25-57) plus the tensor algebra around them.  The shim only
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

m2d_desc describe(const Tensor& x, const Tensor& AT, bool flip) {
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
  d.flags = flip ? M2D_FLAG_FLIP : 0;
  return d;
}

void expect(const Tensor& t, const char* name, const Tensor& x, at::IntArrayRef shape) {
  TORCH_CHECK(t.device() == x.device(), "m2dscan: ", name, " is on ", t.device(), ", x on ", x.device());
  TORCH_CHECK(t.scalar_type() == x.scalar_type(), "m2dscan: ", name, " has dtype ", t.scalar_type(),
              ", x has ", x.scalar_type(), " (all tensors share one dtype)");
  TORCH_CHECK(t.sizes() == shape, "m2dscan: ", name, " has shape ", t.sizes(), ", expected ", shape);
  TORCH_CHECK(t.is_contiguous(), "m2dscan: ", name, " must be contiguous");
}

void expect_all(const m2d_desc& d, const Tensor& x, const Tensor& dT, const Tensor& dL, const Tensor& AT,
                const Tensor& AL, const Tensor& BT, const Tensor& BL, const Tensor& C, const Tensor& D) {
  TORCH_CHECK(x.is_cuda(), "m2dscan: tensors must live on the GPU");
  TORCH_CHECK(x.is_contiguous(), "m2dscan: x must be contiguous");
  const int64_t B = d.B, H = d.H, W = d.W, E = d.E, N = d.N;
  expect(dT, "deltaT", x, {B, H, W, E});
  expect(dL, "deltaL", x, {B, H, W, E});
  expect(AT, "AT", x, {E, N});
  expect(AL, "AL", x, {E, N});
  expect(BT, "BT", x, {B, H, W, N});
  expect(BL, "BL", x, {B, H, W, N});
  expect(C, "C", x, {B, H, W, N});
  expect(D, "D", x, {E});
}

void check(int status) { TORCH_CHECK(status == M2D_OK, "m2dscan: ", m2d_status_str(status), " (status ", status, ")"); }

Tensor bytes(size_t n, const Tensor& like) {
  return at::empty({static_cast<int64_t>(n > 0 ? n : 1)}, like.options().dtype(at::kByte));
}

std::tuple<Tensor, Tensor> scan_fwd(const Tensor& x, const Tensor& dT, const Tensor& dL, const Tensor& AT,
                                    const Tensor& AL, const Tensor& BT, const Tensor& BL, const Tensor& C,
                                    const Tensor& D, bool save_ckpt, bool flip) {
  const m2d_desc d = describe(x, AT, flip);
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
                             const Tensor& ckpt, bool flip) {
  const m2d_desc d = describe(x, AT, flip);
  expect_all(d, x, dT, dL, AT, AL, BT, BL, C, D);
  expect(dy, "dy", x, x.sizes());
  check(m2d_desc_check(&d));
  const bool have = ckpt.numel() > 1;   // a 1-byte tensor stands for "no checkpoints"
  if (have) {
    TORCH_CHECK(ckpt.device() == x.device() && ckpt.scalar_type() == at::kByte && ckpt.is_contiguous(),
                "m2dscan: ckpt must be the byte tensor returned by scan_fwd");
  }
  c10::DeviceGuard guard(x.device());
  std::vector<Tensor> g = {at::empty_like(x),  at::empty_like(dT), at::empty_like(dL), at::empty_like(AT), at::empty_like(AL),
                           at::empty_like(BT), at::empty_like(BL), at::empty_like(C),  at::empty_like(D)};
  Tensor ws = bytes(m2d_scan_workspace_bytes(&d, M2D_PASS_BWD, have), x);
  hipStream_t st = c10::hip::getCurrentHIPStream(x.device().index()).stream();
  check(m2d_scan_bwd(&d, x.data_ptr(), dT.data_ptr(), dL.data_ptr(), AT.data_ptr(), AL.data_ptr(), BT.data_ptr(),
                     BL.data_ptr(), C.data_ptr(), D.data_ptr(), dy.data_ptr(), have ? ckpt.data_ptr() : nullptr,
                     have ? static_cast<size_t>(ckpt.numel()) : 0, g[0].data_ptr(), g[1].data_ptr(), g[2].data_ptr(),
                     g[3].data_ptr(), g[4].data_ptr(), g[5].data_ptr(), g[6].data_ptr(), g[7].data_ptr(),
                     g[8].data_ptr(), ws.data_ptr(), static_cast<size_t>(ws.numel()), st));
  return g;
}

int64_t abi_version() { return m2d_version(); }

}  // namespace

TORCH_LIBRARY(m2dscan, m) {
  m.def("scan_fwd(Tensor x, Tensor deltaT, Tensor deltaL, Tensor AT, Tensor AL, Tensor BT, Tensor BL, Tensor C, "
        "Tensor D, bool save_ckpt, bool flip) -> (Tensor, Tensor)");
  m.def("scan_bwd(Tensor x, Tensor deltaT, Tensor deltaL, Tensor AT, Tensor AL, Tensor BT, Tensor BL, Tensor C, "
        "Tensor D, Tensor dy, Tensor ckpt, bool flip) -> Tensor[]");
  m.def("abi_version() -> int", &abi_version);
}

TORCH_LIBRARY_IMPL(m2dscan, CUDA, m) {   // ROCm devices dispatch under the CUDA key
  m.impl("scan_fwd", &scan_fwd);
  m.impl("scan_bwd", &scan_bwd);
}

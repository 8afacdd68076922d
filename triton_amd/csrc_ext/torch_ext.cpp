// PyTorch-ROCm extension over the C ABI of include/mi355_kernels.h: the analogue of the reference's
// generated launcher (third_party/amd/backend/driver.py:326-377), which pulls pointers out of the
// tensor objects (`data_ptr()`, :285-323), takes the stream the caller's framework is on
// (python/triton/runtime/jit.py:588-589 passes torch's current stream) and launches.  Here: tensor
// checks, sizes / strides / dtypes read off the at::Tensor, c10::hip::getCurrentHIPStream(), one C call.
// No device code in this file and no logic beyond argument marshalling: every status of the C ABI
// becomes the exception the reference raises for the same condition (RuntimeError "Triton Error [HIP]"
// for launch failures, :258-269; ValueError for pointers the device cannot reach, :313-317).
#include <torch/extension.h>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>

#include <stdexcept>
#include <string>

#include "../../include/mi355_kernels.h"

namespace {

int abi_dtype(const at::Tensor& t) {
  switch (t.scalar_type()) {
    case at::kHalf: return MI355_F16;
    case at::kBFloat16: return MI355_BF16;
    case at::kFloat8_e4m3fn: return MI355_F8E4M3;
    case at::kFloat8_e5m2: return MI355_F8E5M2;
    case at::kFloat: return MI355_F32;
    default: throw std::invalid_argument(std::string("unsupported dtype ") + c10::toString(t.scalar_type()));
  }
}

void on_device(const at::Tensor& t, int idx) {
  if (!t.is_cuda())
    throw std::invalid_argument("Pointer argument (at " + std::to_string(idx) + ") cannot be accessed from Triton (cpu tensor?)");
}

void check(int rc, const char* what) {
  if (rc == 0) return;
  const std::string msg = mi355_strerror(rc);
  if (rc > 0)
    throw std::runtime_error("Triton Error [HIP]:  Code: " + std::to_string(rc) + ", Messsage: " + msg + " (" + what + ")");
  throw std::invalid_argument(std::string(what) + ": " + msg + " (code " + std::to_string(rc) + ")");
}

// The C library launches on the CURRENT device: every operator makes its first tensor's device current for the call.
// (the generic guard: it resolves the implementation registered for the tensor's device type, which on ROCm builds of
// torch is the HIP one under the name "cuda")
using DeviceGuard = c10::DeviceGuard;

void* stream_of(const at::Tensor& t) { return (void*)c10::hip::getCurrentHIPStream(t.device().index()).stream(); }

const float* scale_ptr(const c10::optional<at::Tensor>& s) {
  if (!s.has_value()) return nullptr;
  TORCH_CHECK(s->scalar_type() == at::kFloat && s->numel() == 1, "scales are one fp32 value per tensor");
  on_device(*s, -1);
  return s->data_ptr<float>();
}

// C = act((a_scale * b_scale) * A @ B [+ D]) [row softmax]; `add` is already broadcast to [M, N] (zero strides)
void gemm(const at::Tensor& a, const at::Tensor& b, at::Tensor& c, int64_t activation,
          const c10::optional<at::Tensor>& a_scale, const c10::optional<at::Tensor>& b_scale,
          const c10::optional<at::Tensor>& add, bool softmax) {
  TORCH_CHECK(a.dim() == 2 && b.dim() == 2 && c.dim() == 2 && a.size(1) == b.size(0), "Incompatible dimensions");
  on_device(a, 0); on_device(b, 1); on_device(c, 2);
  const DeviceGuard guard(a.device());
  const int M = (int)a.size(0), K = (int)a.size(1), N = (int)b.size(1);
  int rc;
  if (!add.has_value() && !softmax) {
    rc = mi355_gemm(a.data_ptr(), b.data_ptr(), c.data_ptr(), M, N, K, a.stride(0), a.stride(1), b.stride(0), b.stride(1),
                    c.stride(0), c.stride(1), abi_dtype(a), abi_dtype(c), scale_ptr(a_scale), scale_ptr(b_scale),
                    (int)activation, stream_of(a));
    check(rc, "mi355_gemm");
    return;
  }
  const void* d = nullptr;
  int64_t dsm = 0, dsn = 0;
  int ddt = 0;
  if (add.has_value()) {
    on_device(*add, 3);
    d = add->data_ptr(); dsm = add->stride(0); dsn = add->stride(1); ddt = abi_dtype(*add);
  }
  rc = mi355_gemm_epilogue(a.data_ptr(), b.data_ptr(), c.data_ptr(), M, N, K, a.stride(0), a.stride(1), b.stride(0), b.stride(1),
                           c.stride(0), c.stride(1), abi_dtype(a), abi_dtype(c), scale_ptr(a_scale), scale_ptr(b_scale),
                           d, dsm, dsn, ddt, (int)activation, softmax ? 1 : 0, stream_of(a));
  check(rc, "mi355_gemm_epilogue");
}

void mx_gemm(const at::Tensor& a, const at::Tensor& sa, const at::Tensor& b, const at::Tensor& sb, at::Tensor& c, int64_t fmt, int64_t K) {
  on_device(a, 0); on_device(sa, 1); on_device(b, 2); on_device(sb, 3); on_device(c, 4);
  TORCH_CHECK(a.dim() == 2 && b.dim() == 2 && sa.dim() == 2 && sb.dim() == 2 && c.dim() == 2, "MX operands, scales and result are matrices");
  const DeviceGuard guard(a.device());
  const int rc = mi355_mx_gemm((const uint8_t*)a.data_ptr(), (const uint8_t*)sa.data_ptr(), (const uint8_t*)b.data_ptr(),
                               (const uint8_t*)sb.data_ptr(), c.data_ptr(), (int)a.size(0), (int)b.size(0), (int)K, (int)fmt,
                               abi_dtype(c), a.stride(0), b.stride(0), sa.stride(0), sb.stride(0), c.stride(0), stream_of(a));
  check(rc, "mi355_mx_gemm");
}

void strides4(const at::Tensor& t, int64_t (&s)[4]) {
  TORCH_CHECK(t.dim() == 4, "attention tensors are [Z, H, N_CTX, D]");
  for (int i = 0; i < 4; i++) s[i] = t.stride(i);
}

void attn_fwd(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v, at::Tensor& o, at::Tensor& M, double sm_scale, bool causal) {
  on_device(q, 0); on_device(k, 1); on_device(v, 2); on_device(o, 3); on_device(M, 4);
  const DeviceGuard guard(q.device());
  int64_t sq[4], sk[4], sv[4], so[4];
  strides4(q, sq); strides4(k, sk); strides4(v, sv); strides4(o, so);
  const int rc = mi355_attn_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), M.data_ptr<float>(), (int)q.size(0),
                                (int)q.size(1), (int)q.size(2), (int)q.size(3), sq, sk, sv, so, (float)sm_scale, causal ? 1 : 0,
                                abi_dtype(q), stream_of(q));
  check(rc, "mi355_attn_fwd");
}

void attn_bwd(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v, const at::Tensor& o, const at::Tensor& d_o,
              const at::Tensor& M, at::Tensor& delta, at::Tensor& dq, at::Tensor& dk, at::Tensor& dv, double sm_scale, bool causal) {
  on_device(q, 0); on_device(k, 1); on_device(v, 2); on_device(o, 3); on_device(d_o, 4); on_device(M, 5);
  on_device(delta, 6); on_device(dq, 7); on_device(dk, 8); on_device(dv, 9);
  const DeviceGuard guard(q.device());
  int64_t s[4], so[4];
  strides4(q, s); strides4(o, so);
  const int Z = (int)q.size(0), H = (int)q.size(1), N = (int)q.size(2), D = (int)q.size(3);
  void* stream = stream_of(q);
  int rc = mi355_attn_bwd_preprocess(o.data_ptr(), d_o.data_ptr(), delta.data_ptr<float>(), Z, H, N, D, so, abi_dtype(q), stream);
  check(rc, "mi355_attn_bwd_preprocess");
  rc = mi355_attn_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), d_o.data_ptr(), M.data_ptr<float>(), delta.data_ptr<float>(),
                      dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), Z, H, N, D, s, (float)sm_scale, causal ? 1 : 0, abi_dtype(q), stream);
  check(rc, "mi355_attn_bwd");
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.doc() = "PyTorch-ROCm extension over the MI355X kernel library's C ABI";
  m.def("gemm", &gemm);
  m.def("mx_gemm", &mx_gemm);
  m.def("attn_fwd", &attn_fwd);
  m.def("attn_bwd", &attn_bwd);
}

// PyTorch (ROCm) face of the C ABI: registers the reference's three operators, with
// the reference's schemas, under torch.ops.matgptq_cuda (and the reference's C++
// namespace name _matgptq_cuda_C), plus additive extensions.  Counterpart of
// inference_lib/matgptq_cuda/csrc/bindings.cpp:43-220 and of the Python custom_op
// layer inference_lib/matgptq_cuda/__init__.py:5-63.  Everything here is argument
// checking, allocation through torch's caching allocator and a call into
// include/matgptq_abi.h on torch's current stream; no arithmetic happens in this file.
#include <ATen/ATen.h>
#include <ATen/hip/HIPContext.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/extension.h>
#include <torch/library.h>

#include "../../include/matgptq_abi.h"

namespace {

using torch::Tensor;

void check_bits_group(int64_t bitwidth, int64_t group_size, int64_t n_in_features) {
  // messages of the reference (bindings.cpp:55-59)
  TORCH_CHECK(bitwidth == 2 || bitwidth == 3 || bitwidth == 4 || bitwidth == 6 || bitwidth == 8,
              "bitwidth must be one of {2, 3, 4, 6, 8}");
  TORCH_CHECK(group_size == -1 || group_size == 32 || group_size == 128,
              "group_size must be one of {-1, 32, 128}");
  if (group_size != -1) {
    TORCH_CHECK(n_in_features % group_size == 0,
                "group_size must divide n_in_features. Got group_size=", group_size,
                ", n_in_features=", n_in_features);
  }
}

// The reference needs n_in_features % 64 == 0 (utils.cpp:174-184).  Here: a multiple of 128, or
// (where the group size divides it: 32 and -1) such a multiple plus 64; `whole_tiles`: the
// master-resident planes take multiples of 128 only.
void check_tiling(int64_t n_out_features, int64_t n_in_features, bool whole_tiles = false) {
  TORCH_CHECK(n_out_features > 0 && n_out_features % 16 == 0,
              "n_out_features must be a positive multiple of 16, got ", n_out_features);
  if (whole_tiles) {
    TORCH_CHECK(n_in_features > 0 && n_in_features % 128 == 0,
                "n_in_features must be a positive multiple of 128, got ", n_in_features);
  } else {
    TORCH_CHECK(n_in_features > 0 && (n_in_features % 128 == 0 || (n_in_features % 128 == 64 && n_in_features >= 192)),
                "n_in_features must be a positive multiple of 128, or at least 192 and a multiple of 128 plus 64, got ",
                n_in_features);
  }
}

void check_abi(int code, const char* what) {
  TORCH_CHECK(code == MATGPTQ_OK, what, ": ", matgptq_strerror(code));
}

at::Device target_device(const Tensor& t) {
  // The reference sends the result to the GPU of the input, or to the current GPU
  // when the input lives on the host (bindings.cpp:62,83).
  if (t.is_cuda()) return t.device();
  return at::Device(at::kCUDA, at::cuda::current_device());
}

void* stream_of(const at::Device& dev) {
  return static_cast<void*>(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(dev.index()).stream());
}

// pack_matgptq_qweights (bindings.cpp:43-84).  `slice_from_master` is the additive part:
// 0 = codes are already sliced (the reference's contract), 1 = 8-bit master codes.
Tensor pack_impl(const Tensor& qweights, int64_t n_out_features, int64_t n_in_features,
                 int64_t bitwidth, int64_t group_size, int64_t feature_flag,
                 int64_t slice_from_master) {
  (void)feature_flag;  // the packed layout does not depend on the activation dtype
  TORCH_CHECK(qweights.dtype() == torch::kUInt8, "qweights must be uint8");
  TORCH_CHECK(qweights.is_contiguous(), "qweights must be contiguous");
  TORCH_CHECK(qweights.dim() == 2, "qweights must be 2D (n_out_features, n_in_features)");
  TORCH_CHECK(qweights.size(0) == n_out_features, "n_out_features does not match qweights.size(0)");
  TORCH_CHECK(qweights.size(1) == n_in_features, "n_in_features does not match qweights.size(1)");
  check_bits_group(bitwidth, group_size, n_in_features);
  check_tiling(n_out_features, n_in_features);
  const at::Device dev = target_device(qweights);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(dev);
  const int64_t words = bitwidth * n_out_features * n_in_features / 32;
  Tensor out = torch::empty({words}, torch::dtype(torch::kUInt32).device(dev));
  if (qweights.is_cuda()) {
    check_abi(matgptq_pack_device(qweights.data_ptr<uint8_t>(), n_out_features, n_in_features,
                                  (int)bitwidth, (int)slice_from_master,
                                  static_cast<uint32_t*>(out.data_ptr()), stream_of(dev)),
              "pack_matgptq_qweights");
  } else {
    Tensor host = torch::empty({words}, torch::dtype(torch::kUInt32).device(torch::kCPU));
    check_abi(matgptq_pack_host(qweights.data_ptr<uint8_t>(), n_out_features, n_in_features,
                                (int)bitwidth, (int)slice_from_master,
                                static_cast<uint32_t*>(host.data_ptr())),
              "pack_matgptq_qweights");
    out.copy_(host);
  }
  return out;
}

Tensor pack_matgptq_qweights(const Tensor& qweights, int64_t n_out_features, int64_t n_in_features,
                             int64_t bitwidth, int64_t group_size, int64_t feature_flag) {
  return pack_impl(qweights, n_out_features, n_in_features, bitwidth, group_size, feature_flag, 0);
}

Tensor pack_matgptq_master(const Tensor& qweights, int64_t n_out_features, int64_t n_in_features,
                           int64_t bitwidth, int64_t group_size, int64_t feature_flag) {
  return pack_impl(qweights, n_out_features, n_in_features, bitwidth, group_size, feature_flag, 1);
}

// reorder_matgptq_scales (bindings.cpp:86-142): same shape and dtype out, on the GPU.
Tensor reorder_matgptq_scales(const Tensor& scales, int64_t n_out_features, int64_t n_in_features,
                              int64_t group_size) {
  TORCH_CHECK(scales.is_contiguous(), "scales must be contiguous");
  TORCH_CHECK(scales.dim() == 2, "qweights must be 2D (n_out_features, n_in_features)");
  TORCH_CHECK(scales.dtype() == torch::kFloat16 || scales.dtype() == torch::kBFloat16,
              "scales must be float16 or bfloat16");
  check_bits_group(8, group_size, n_in_features);
  check_tiling(n_out_features, n_in_features);
  const int64_t groups = group_size == -1 ? 1 : n_in_features / group_size;
  TORCH_CHECK(scales.size(0) == n_out_features && scales.size(1) == groups,
              "scales must have shape (n_out_features, n_in_features / group_size)");
  const at::Device dev = target_device(scales);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(dev);
  Tensor out = torch::empty(scales.sizes(), scales.options().device(dev));
  if (scales.is_cuda()) {
    check_abi(matgptq_reorder_scales_device(static_cast<const uint16_t*>(scales.data_ptr()),
                                            n_out_features, n_in_features, (int)group_size,
                                            static_cast<uint16_t*>(out.data_ptr()), stream_of(dev)),
              "reorder_matgptq_scales");
  } else {
    Tensor host = torch::empty_like(scales);
    check_abi(matgptq_reorder_scales_host(static_cast<const uint16_t*>(scales.data_ptr()),
                                          n_out_features, n_in_features, (int)group_size,
                                          static_cast<uint16_t*>(host.data_ptr())),
              "reorder_matgptq_scales");
    out.copy_(host);
  }
  return out;
}

// matmul_matgptq (bindings.cpp:146-191) and its zero-point extension.
// `master`: `weights` are master-resident bit planes (N*K/4 words) instead of a pre-sliced tensor
Tensor matmul_impl(const Tensor& input, const Tensor& weights, const Tensor& scales,
                   const c10::optional<Tensor>& zeros, int64_t n_out_features,
                   int64_t n_in_features, int64_t bitwidth, int64_t group_size,
                   int64_t feature_flag, bool master = false) {
  TORCH_CHECK(input.is_cuda() && weights.is_cuda() && scales.is_cuda(),
              "matmul_matgptq: input, matgptq_weights and matgptq_scales must be GPU tensors");
  TORCH_CHECK(input.device() == weights.device() && input.device() == scales.device(),
              "matmul_matgptq: input, matgptq_weights and matgptq_scales must be on the same GPU");
  TORCH_CHECK(weights.dtype() == torch::kUInt32, "matgptq_weights must be uint32");
  TORCH_CHECK(weights.is_contiguous(), "matgptq_weights must be contiguous");
  TORCH_CHECK(weights.dim() == 1, "qweights must be 1D");
  check_bits_group(bitwidth, group_size, n_in_features);
  check_tiling(n_out_features, n_in_features);
  TORCH_CHECK(weights.size(0) == (master ? 8 : bitwidth) * n_out_features * n_in_features / 32,
              "matgptq_weights has the wrong size");
  const bool bf16 = (feature_flag & MATGPTQ_FLAG_BF16) != 0;
  // the reference trusts the flag (bindings.cpp:171-174); a mismatch is reported here
  const auto want = bf16 ? torch::kBFloat16 : torch::kFloat16;
  const char* want_name = bf16 ? "bfloat16 (feature_flag bit 1 is set)" : "float16 (feature_flag bit 1 is clear)";
  TORCH_CHECK(input.dtype() == want, "matmul_matgptq: input must be ", want_name);
  TORCH_CHECK(scales.dtype() == want, "matmul_matgptq: matgptq_scales must be ", want_name);
  TORCH_CHECK(input.dim() >= 2 && input.size(-1) == n_in_features,
              "matmul_matgptq: input must be (..., batch, n_in_features)");
  // the reference reads the input as if it were contiguous (bindings.cpp:171-186): a strided
  // view (a slice of a fused projection, a transposed batch) is compacted first
  const Tensor input_c = input.contiguous();
  const int64_t groups = group_size == -1 ? 1 : n_in_features / group_size;
  TORCH_CHECK(scales.is_contiguous() && scales.numel() == n_out_features * groups,
              "matgptq_scales has the wrong size");
  const void* zeros_ptr = nullptr;
  if (zeros.has_value()) {
    const Tensor& z = *zeros;
    TORCH_CHECK(z.is_cuda() && z.device() == input.device(), "matgptq_zeros must be on the GPU of the input");
    TORCH_CHECK(z.dtype() == want, "matgptq_zeros must be ", want_name);
    TORCH_CHECK(z.is_contiguous() && z.numel() == n_out_features * groups,
                "matgptq_zeros has the wrong size");
    zeros_ptr = z.data_ptr();
  }
  // The reference returns (input.size(-2), N) and reads exactly that many rows
  // (bindings.cpp:171-174); leading dimensions are folded into the batch here, which
  // agrees with it for 2-D inputs and for a leading dimension of one.
  const int64_t m = input.numel() / n_in_features;
  const at::Device dev = input.device();
  c10::hip::HIPGuardMasqueradingAsCUDA guard(dev);
  Tensor out = torch::empty({m, n_out_features}, input.options());
  if (m == 0) return out;
  const uint32_t flags = (uint32_t)feature_flag | MATGPTQ_FLAG_ASYNC;
  int code;
  if (master) {
    // shapes outside the kernel that reads the planes itself need the pre-sliced tensor in a
    // workspace: taken from torch's caching allocator (capturable like the output)
    const size_t ws_bytes = matgptq_gemm_master_workspace_bytes((int)bitwidth, (int)group_size, n_out_features,
                                                               n_in_features, m, flags);
    Tensor ws;
    if (ws_bytes > 0) ws = torch::empty({(int64_t)ws_bytes}, input.options().dtype(torch::kUInt8));
    code = matgptq_gemm_master((int)bitwidth, (int)group_size, n_out_features, n_in_features, m,
                               weights.data_ptr(), scales.data_ptr(), zeros_ptr, input_c.data_ptr(),
                               out.data_ptr(), ws_bytes > 0 ? ws.data_ptr() : nullptr, ws_bytes,
                               stream_of(dev), flags);
  } else {
    code = matgptq_gemm((int)bitwidth, (int)group_size, n_out_features, n_in_features, m,
                        weights.data_ptr(), scales.data_ptr(), zeros_ptr, input_c.data_ptr(),
                        out.data_ptr(), stream_of(dev), flags);
  }
  check_abi(code, "matmul_matgptq");
  if (!(feature_flag & MATGPTQ_FLAG_ASYNC)) {
    // SYNC mode of the reference: the call returns after the kernel (matgptq_gemm.cu:1060-1062)
    c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(dev.index()).synchronize();
  }
  return out;
}

Tensor matmul_matgptq(const Tensor& input, const Tensor& weights, const Tensor& scales,
                      int64_t n_out_features, int64_t n_in_features, int64_t bitwidth,
                      int64_t group_size, int64_t feature_flag) {
  return matmul_impl(input, weights, scales, c10::nullopt, n_out_features, n_in_features, bitwidth,
                     group_size, feature_flag);
}

Tensor matmul_matgptq_zp(const Tensor& input, const Tensor& weights, const Tensor& scales,
                         const Tensor& zeros, int64_t n_out_features, int64_t n_in_features,
                         int64_t bitwidth, int64_t group_size, int64_t feature_flag) {
  return matmul_impl(input, weights, scales, zeros, n_out_features, n_in_features, bitwidth,
                     group_size, feature_flag);
}

// ---- master-resident codes (additive; see include/matgptq_abi.h) ----
Tensor matmul_matgptq_master(const Tensor& input, const Tensor& planes, const Tensor& scales,
                             const c10::optional<Tensor>& zeros, int64_t n_out_features,
                             int64_t n_in_features, int64_t bitwidth, int64_t group_size,
                             int64_t feature_flag) {
  return matmul_impl(input, planes, scales, zeros, n_out_features, n_in_features, bitwidth, group_size,
                     feature_flag, true);
}

Tensor pack_matgptq_master_resident(const Tensor& qweights) {
  TORCH_CHECK(qweights.dtype() == torch::kUInt8, "qweights must be uint8");
  TORCH_CHECK(qweights.is_contiguous(), "qweights must be contiguous");
  TORCH_CHECK(qweights.dim() == 2, "qweights must be 2D (n_out_features, n_in_features)");
  const int64_t n = qweights.size(0), k = qweights.size(1);
  check_tiling(n, k, true);
  const at::Device dev = target_device(qweights);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(dev);
  const int64_t words = n * k / 4;
  Tensor out = torch::empty({words}, torch::dtype(torch::kUInt32).device(dev));
  if (qweights.is_cuda()) {
    check_abi(matgptq_pack_master_device(qweights.data_ptr<uint8_t>(), n, k, static_cast<uint32_t*>(out.data_ptr()),
                                         stream_of(dev)),
              "pack_matgptq_master_resident");
  } else {
    Tensor host = torch::empty({words}, torch::dtype(torch::kUInt32).device(torch::kCPU));
    check_abi(matgptq_pack_master_host(qweights.data_ptr<uint8_t>(), n, k, static_cast<uint32_t*>(host.data_ptr())),
              "pack_matgptq_master_resident");
    out.copy_(host);
  }
  return out;
}

Tensor unpack_matgptq_master_resident(const Tensor& planes, int64_t n_out_features, int64_t n_in_features,
                                      int64_t bitwidth) {
  TORCH_CHECK(planes.dtype() == torch::kUInt32 && planes.dim() == 1 && planes.is_contiguous(),
              "master planes must be a contiguous 1D uint32 tensor");
  check_bits_group(bitwidth, -1, n_in_features);
  check_tiling(n_out_features, n_in_features, true);
  TORCH_CHECK(planes.size(0) == n_out_features * n_in_features / 4, "master planes have the wrong size");
  Tensor out = torch::empty({n_out_features, n_in_features}, planes.options().dtype(torch::kUInt8));
  if (planes.is_cuda()) {
    c10::hip::HIPGuardMasqueradingAsCUDA guard(planes.device());
    check_abi(matgptq_unpack_master_device(static_cast<const uint32_t*>(planes.data_ptr()), n_out_features,
                                           n_in_features, (int)bitwidth, out.data_ptr<uint8_t>(),
                                           stream_of(planes.device())),
              "unpack_matgptq_master_resident");
  } else {
    check_abi(matgptq_unpack_master_host(static_cast<const uint32_t*>(planes.data_ptr()), n_out_features,
                                         n_in_features, (int)bitwidth, out.data_ptr<uint8_t>()),
              "unpack_matgptq_master_resident");
  }
  return out;
}

// Debug / test helpers: the codes and the dense weight a packed tensor stands for.
Tensor unpack_matgptq_qweights(const Tensor& weights, int64_t n_out_features, int64_t n_in_features,
                               int64_t bitwidth) {
  TORCH_CHECK(weights.dtype() == torch::kUInt32 && weights.dim() == 1 && weights.is_contiguous(),
              "matgptq_weights must be a contiguous 1D uint32 tensor");
  check_bits_group(bitwidth, -1, n_in_features);
  check_tiling(n_out_features, n_in_features);
  TORCH_CHECK(weights.size(0) == bitwidth * n_out_features * n_in_features / 32,
              "matgptq_weights has the wrong size");
  Tensor out = torch::empty({n_out_features, n_in_features}, weights.options().dtype(torch::kUInt8));
  if (weights.is_cuda()) {
    c10::hip::HIPGuardMasqueradingAsCUDA guard(weights.device());
    check_abi(matgptq_unpack_device(static_cast<const uint32_t*>(weights.data_ptr()), n_out_features,
                                    n_in_features, (int)bitwidth, out.data_ptr<uint8_t>(),
                                    stream_of(weights.device())),
              "unpack_matgptq_qweights");
  } else {
    check_abi(matgptq_unpack_host(static_cast<const uint32_t*>(weights.data_ptr()), n_out_features,
                                  n_in_features, (int)bitwidth, out.data_ptr<uint8_t>()),
              "unpack_matgptq_qweights");
  }
  return out;
}

Tensor slice_matgptq_master(const Tensor& master, int64_t bitwidth) {
  TORCH_CHECK(master.dtype() == torch::kUInt8 && master.is_contiguous(),
              "master codes must be a contiguous uint8 tensor");
  TORCH_CHECK(master.is_cuda(), "slice_matgptq_master: master codes must be on the GPU");
  check_bits_group(bitwidth, -1, 128);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(master.device());
  Tensor out = torch::empty_like(master);
  check_abi(matgptq_slice_device(master.data_ptr<uint8_t>(), master.numel(), (int)bitwidth,
                                 out.data_ptr<uint8_t>(), stream_of(master.device())),
            "slice_matgptq_master");
  return out;
}

Tensor dequantize_matgptq(const Tensor& weights, const Tensor& scales,
                          const c10::optional<Tensor>& zeros, int64_t n_out_features,
                          int64_t n_in_features, int64_t bitwidth, int64_t group_size) {
  TORCH_CHECK(weights.is_cuda() && scales.is_cuda(), "dequantize_matgptq: GPU tensors expected");
  TORCH_CHECK(weights.dtype() == torch::kUInt32 && weights.dim() == 1 && weights.is_contiguous(),
              "matgptq_weights must be a contiguous 1D uint32 tensor");
  check_bits_group(bitwidth, group_size, n_in_features);
  check_tiling(n_out_features, n_in_features);
  TORCH_CHECK(weights.size(0) == bitwidth * n_out_features * n_in_features / 32,
              "matgptq_weights has the wrong size");
  TORCH_CHECK(scales.dtype() == torch::kFloat16 && scales.is_contiguous(), "matgptq_scales must be contiguous float16");
  const int64_t groups = group_size == -1 ? 1 : n_in_features / group_size;
  TORCH_CHECK(scales.numel() == n_out_features * groups, "matgptq_scales has the wrong size");
  const void* zp = nullptr;
  if (zeros.has_value()) {
    TORCH_CHECK(zeros->is_cuda() && zeros->dtype() == torch::kFloat16 && zeros->is_contiguous() &&
                    zeros->numel() == n_out_features * groups,
                "matgptq_zeros must be a contiguous float16 GPU tensor of the scales' size");
    zp = zeros->data_ptr();
  }
  c10::hip::HIPGuardMasqueradingAsCUDA guard(weights.device());
  Tensor out = torch::empty({n_out_features, n_in_features}, scales.options());
  check_abi(matgptq_dequantize_device((int)bitwidth, (int)group_size, n_out_features, n_in_features,
                                      weights.data_ptr(), scales.data_ptr(), zp, out.data_ptr(),
                                      stream_of(weights.device())),
            "dequantize_matgptq");
  return out;
}

std::string describe_plan(int64_t bitwidth, int64_t group_size, int64_t n_out_features,
                          int64_t n_in_features, int64_t batch, bool has_zeros, int64_t flags) {
  char buf[160];
  check_abi(matgptq_describe_plan((int)bitwidth, (int)group_size, n_out_features, n_in_features,
                                  batch, has_zeros ? 1 : 0, (uint32_t)flags, buf, sizeof(buf)),
            "describe_plan");
  return std::string(buf);
}

constexpr const char* kPackSchema =
    "(Tensor qweights, int n_out_features, int n_in_features, int bitwidth, int group_size, "
    "int feature_flag) -> Tensor";
constexpr const char* kReorderSchema =
    "(Tensor scales, int n_out_features, int n_in_features, int group_size) -> Tensor";
constexpr const char* kMatmulSchema =
    "(Tensor input, Tensor matgptq_weights, Tensor matgptq_scales, int n_out_features, "
    "int n_in_features, int bitwidth, int group_size, int feature_flag) -> Tensor";

void define_ops(torch::Library& m) {
  // the three schemas of the reference (bindings.cpp:198-200)
  m.def((std::string("pack_matgptq_qweights") + kPackSchema).c_str());
  m.def((std::string("reorder_matgptq_scales") + kReorderSchema).c_str());
  m.def((std::string("matmul_matgptq") + kMatmulSchema).c_str());
}

}  // namespace

// Namespace the reference's Python layer exposes (torch.ops.matgptq_cuda.*), extended.
TORCH_LIBRARY(matgptq_cuda, m) {
  define_ops(m);
  m.def((std::string("pack_matgptq_master") + kPackSchema).c_str());
  m.def("matmul_matgptq_zp(Tensor input, Tensor matgptq_weights, Tensor matgptq_scales, "
        "Tensor matgptq_zeros, int n_out_features, int n_in_features, int bitwidth, int group_size, "
        "int feature_flag) -> Tensor");
  m.def("unpack_matgptq_qweights(Tensor matgptq_weights, int n_out_features, int n_in_features, "
        "int bitwidth) -> Tensor");
  m.def("slice_matgptq_master(Tensor master, int bitwidth) -> Tensor");
  m.def("pack_matgptq_master_resident(Tensor qweights) -> Tensor");
  m.def("unpack_matgptq_master_resident(Tensor planes, int n_out_features, int n_in_features, "
        "int bitwidth) -> Tensor");
  m.def("matmul_matgptq_master(Tensor input, Tensor planes, Tensor matgptq_scales, Tensor? matgptq_zeros, "
        "int n_out_features, int n_in_features, int bitwidth, int group_size, int feature_flag) -> Tensor");
  m.def("dequantize_matgptq(Tensor matgptq_weights, Tensor matgptq_scales, Tensor? matgptq_zeros, "
        "int n_out_features, int n_in_features, int bitwidth, int group_size) -> Tensor");
}

// Pack / reorder take host or device tensors, so they are registered for every backend
// (the reference reaches its C++ function without the dispatcher for the same reason,
// inference_lib/matgptq_cuda/__init__.py:5-24).
TORCH_LIBRARY_IMPL(matgptq_cuda, CompositeExplicitAutograd, m) {
  m.impl("pack_matgptq_qweights", TORCH_FN(pack_matgptq_qweights));
  m.impl("pack_matgptq_master", TORCH_FN(pack_matgptq_master));
  m.impl("reorder_matgptq_scales", TORCH_FN(reorder_matgptq_scales));
  m.impl("unpack_matgptq_qweights", TORCH_FN(unpack_matgptq_qweights));
  m.impl("pack_matgptq_master_resident", TORCH_FN(pack_matgptq_master_resident));
  m.impl("unpack_matgptq_master_resident", TORCH_FN(unpack_matgptq_master_resident));
}

// On ROCm builds of PyTorch HIP tensors carry the CUDA dispatch key.
TORCH_LIBRARY_IMPL(matgptq_cuda, CUDA, m) {
  m.impl("matmul_matgptq", TORCH_FN(matmul_matgptq));
  m.impl("matmul_matgptq_zp", TORCH_FN(matmul_matgptq_zp));
  m.impl("matmul_matgptq_master", TORCH_FN(matmul_matgptq_master));
  m.impl("slice_matgptq_master", TORCH_FN(slice_matgptq_master));
  m.impl("dequantize_matgptq", TORCH_FN(dequantize_matgptq));
}

// Name of the reference's C++ registration (bindings.cpp:197-207).
TORCH_LIBRARY(_matgptq_cuda_C, m) { define_ops(m); }
TORCH_LIBRARY_IMPL(_matgptq_cuda_C, CompositeExplicitAutograd, m) {
  m.impl("pack_matgptq_qweights", TORCH_FN(pack_matgptq_qweights));
  m.impl("reorder_matgptq_scales", TORCH_FN(reorder_matgptq_scales));
}
TORCH_LIBRARY_IMPL(_matgptq_cuda_C, CUDA, m) { m.impl("matmul_matgptq", TORCH_FN(matmul_matgptq)); }

// Python module with the reference's three pybind names (bindings.cpp:213-220).
PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("pack_matgptq_qweights", &pack_matgptq_qweights, "pack_matgptq_qweights");
  m.def("reorder_matgptq_scales", &reorder_matgptq_scales, "reorder_matgptq_scales");
  m.def("matmul_matgptq", &matmul_matgptq, "matmul_matgptq");
  m.def("matmul_matgptq_zp", &matmul_matgptq_zp, "matmul_matgptq_zp");
  m.def("pack_matgptq_master", &pack_matgptq_master, "pack_matgptq_master");
  m.def("describe_plan", &describe_plan, "describe_plan");
  m.def("abi_version", []() { return matgptq_abi_version(); }, "abi_version");
}

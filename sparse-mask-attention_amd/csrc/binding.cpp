// Python module `sparse_attn_cuda`: a thin pybind11 shim over the C ABI of libsma_hip.so.
//
// It keeps the module name and the two Python-visible signatures of the reference binding
// (csrc/binding.cpp:9-18 `forward`, csrc/binding.cpp:49 `pack_mask`, registered at
// csrc/binding.cpp:68-71) so that python/sparse_attention.py can stay as it is:
//
//   forward(q, k, v, mask_packed, out, lse, scale, is_training) -> None
//   pack_mask(mask) -> int32 Tensor [B, H, N, ceil(N/32)]
//   backward(dout, q, k, v, out, lse, mask_packed, dq, dk, dv, scale) -> None   (called by the
//       reference's Python API, python/sparse_attention.py:91-94, but absent from its binding)
//
// Differences, all on the safe side: `lse` may be None (the reference's own inference wrapper
// passes None, python/sparse_attention.py:170-171); every tensor argument is checked (device,
// dtype, shape, contiguity, head_dim == 64) instead of only `q`; launches go to the current HIP
// stream of q's device under a device guard; a failed launch raises RuntimeError.
// This file is host-only C++ (compiled by g++); all GPU code lives behind include/sma.h.
#include <torch/extension.h>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>

#include "sma.h"

namespace {

void check_status(int st, const char *what)
{
    TORCH_CHECK(st == SMA_OK, what, " failed: ", sma_strerror(st), " (code ", st, ")");
}

void forward(const torch::Tensor &q, const torch::Tensor &k, const torch::Tensor &v,
             const torch::Tensor &mask_packed, torch::Tensor out,
             const c10::optional<torch::Tensor> &lse, double scale, bool is_training)
{
    TORCH_CHECK(q.is_cuda(), "q must be a GPU tensor");
    TORCH_CHECK(q.dim() == 4, "q must be 4D [B, H, N, D]");
    const auto dt = q.scalar_type();
    TORCH_CHECK(dt == at::kHalf || dt == at::kBFloat16, "Unsupported dtype, need BF16 or FP16");
    const int64_t B = q.size(0), H = q.size(1), N = q.size(2), D = q.size(3);
    TORCH_CHECK(D == 64, "head_dim must be 64, got ", D);
    for (const torch::Tensor *t : {&k, &v, static_cast<const torch::Tensor *>(&out)}) {
        TORCH_CHECK(t->device() == q.device(), "q, k, v, out must be on the same device");
        TORCH_CHECK(t->scalar_type() == dt, "q, k, v, out must have the same dtype");
        TORCH_CHECK(t->sizes() == q.sizes(), "q, k, v, out must have the same shape");
        TORCH_CHECK(t->is_contiguous(), "q, k, v, out must be contiguous");
    }
    TORCH_CHECK(q.is_contiguous(), "q must be contiguous");
    const int64_t nw = (N + 31) / 32;
    TORCH_CHECK(mask_packed.device() == q.device(), "mask_packed must be on q's device");
    TORCH_CHECK(mask_packed.scalar_type() == at::kInt, "mask_packed must be int32");
    TORCH_CHECK(mask_packed.dim() == 4 && mask_packed.size(0) == B && mask_packed.size(1) == H &&
                    mask_packed.size(2) == N && mask_packed.size(3) == nw,
                "mask_packed must be [B, H, N, ceil(N/32)]");
    TORCH_CHECK(mask_packed.is_contiguous(), "mask_packed must be contiguous");
    float *lse_ptr = nullptr;
    if (is_training) {
        TORCH_CHECK(lse.has_value() && lse->defined(), "is_training=True needs an lse tensor");
        TORCH_CHECK(lse->device() == q.device() && lse->scalar_type() == at::kFloat &&
                        lse->dim() == 3 && lse->size(0) == B && lse->size(1) == H &&
                        lse->size(2) == N && lse->is_contiguous(),
                    "lse must be a contiguous float32 [B, H, N] tensor on q's device");
        lse_ptr = lse->data_ptr<float>();
    }
    TORCH_CHECK(B <= INT32_MAX && H <= INT32_MAX && N <= INT32_MAX, "extent too large");

    const c10::DeviceGuard guard(q.device());
    hipStream_t stream = c10::hip::getCurrentHIPStream(q.device().index()).stream();
    const int st = sma_attn_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(),
                                reinterpret_cast<const uint32_t *>(mask_packed.data_ptr<int32_t>()),
                                out.data_ptr(), lse_ptr, (int)B, (int)H, (int)N, (int)D,
                                (float)scale, dt == at::kBFloat16 ? SMA_DTYPE_BF16 : SMA_DTYPE_F16,
                                stream);
    check_status(st, "sma_attn_fwd");
}

// backward(dout, q, k, v, out, lse, mask_packed, dq, dk, dv, scale) -> None, the call the
// reference's autograd function makes (python/sparse_attention.py:91-94) to a function its
// binding never had.  dq, dk, dv are overwritten (not accumulated into).
void backward(const torch::Tensor &dout, const torch::Tensor &q, const torch::Tensor &k,
              const torch::Tensor &v, const torch::Tensor &out, const torch::Tensor &lse,
              const torch::Tensor &mask_packed, torch::Tensor dq, torch::Tensor dk,
              torch::Tensor dv, double scale)
{
    TORCH_CHECK(q.is_cuda(), "q must be a GPU tensor");
    TORCH_CHECK(q.dim() == 4, "q must be 4D [B, H, N, D]");
    const auto dt = q.scalar_type();
    TORCH_CHECK(dt == at::kHalf || dt == at::kBFloat16, "Unsupported dtype, need BF16 or FP16");
    const int64_t B = q.size(0), H = q.size(1), N = q.size(2), D = q.size(3);
    TORCH_CHECK(D == 64, "head_dim must be 64, got ", D);
    for (const torch::Tensor *t : {&dout, &q, &k, &v, &out, static_cast<const torch::Tensor *>(&dq),
                                   static_cast<const torch::Tensor *>(&dk),
                                   static_cast<const torch::Tensor *>(&dv)}) {
        TORCH_CHECK(t->device() == q.device(), "dout, q, k, v, out, dq, dk, dv must be on the same device");
        TORCH_CHECK(t->scalar_type() == dt, "dout, q, k, v, out, dq, dk, dv must have the same dtype");
        TORCH_CHECK(t->sizes() == q.sizes(), "dout, q, k, v, out, dq, dk, dv must have the same shape");
        TORCH_CHECK(t->is_contiguous(), "dout, q, k, v, out, dq, dk, dv must be contiguous");
    }
    const int64_t nw = (N + 31) / 32;
    TORCH_CHECK(mask_packed.device() == q.device() && mask_packed.scalar_type() == at::kInt &&
                    mask_packed.dim() == 4 && mask_packed.size(0) == B && mask_packed.size(1) == H &&
                    mask_packed.size(2) == N && mask_packed.size(3) == nw && mask_packed.is_contiguous(),
                "mask_packed must be a contiguous int32 [B, H, N, ceil(N/32)] tensor on q's device");
    TORCH_CHECK(lse.device() == q.device() && lse.scalar_type() == at::kFloat && lse.dim() == 3 &&
                    lse.size(0) == B && lse.size(1) == H && lse.size(2) == N && lse.is_contiguous(),
                "lse must be a contiguous float32 [B, H, N] tensor on q's device");
    TORCH_CHECK(B <= INT32_MAX && H <= INT32_MAX && N <= INT32_MAX, "extent too large");

    const c10::DeviceGuard guard(q.device());
    torch::Tensor delta = torch::empty({B, H, N}, lse.options());      // workspace of the C entry point
    hipStream_t stream = c10::hip::getCurrentHIPStream(q.device().index()).stream();
    const int st = sma_attn_bwd(dout.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                lse.data_ptr<float>(),
                                reinterpret_cast<const uint32_t *>(mask_packed.data_ptr<int32_t>()),
                                dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), delta.data_ptr<float>(),
                                (int)B, (int)H, (int)N, (int)D, (float)scale,
                                dt == at::kBFloat16 ? SMA_DTYPE_BF16 : SMA_DTYPE_F16, stream);
    check_status(st, "sma_attn_bwd");
}

torch::Tensor pack_mask(const torch::Tensor &mask)
{
    TORCH_CHECK(mask.is_cuda(), "mask must be a GPU tensor");
    TORCH_CHECK(mask.dim() == 4, "mask must be 4D [B, H, N, N]");
    TORCH_CHECK(mask.scalar_type() == at::kBool, "mask must be bool");
    TORCH_CHECK(mask.size(2) == mask.size(3), "mask must be [B, H, N, N]");
    const torch::Tensor m = mask.contiguous();
    const int64_t B = m.size(0), H = m.size(1), N = m.size(2);
    TORCH_CHECK(B <= INT32_MAX && H <= INT32_MAX && N <= INT32_MAX, "extent too large");
    const c10::DeviceGuard guard(m.device());
    // Every word is written by the kernel, so no zero-fill is needed.
    torch::Tensor packed = torch::empty({B, H, N, (N + 31) / 32}, m.options().dtype(torch::kInt32));
    hipStream_t stream = c10::hip::getCurrentHIPStream(m.device().index()).stream();
    const int st = sma_pack_mask(reinterpret_cast<const uint8_t *>(m.data_ptr<bool>()),
                                 reinterpret_cast<uint32_t *>(packed.data_ptr<int32_t>()), (int)B,
                                 (int)H, (int)N, stream);
    check_status(st, "sma_pack_mask");
    return packed;
}

}  // namespace

PYBIND11_MODULE(sparse_attn_cuda, m)
{
    m.doc() = "sparse-mask attention for MI355X (gfx950): pybind shim over libsma_hip.so";
    m.def("forward", &forward, "Sparse-mask attention forward", py::arg("q"), py::arg("k"),
          py::arg("v"), py::arg("mask_packed"), py::arg("out"), py::arg("lse"), py::arg("scale"),
          py::arg("is_training"));
    m.def("backward", &backward, "Sparse-mask attention backward (dq, dk, dv are overwritten)",
          py::arg("dout"), py::arg("q"), py::arg("k"), py::arg("v"), py::arg("out"), py::arg("lse"),
          py::arg("mask_packed"), py::arg("dq"), py::arg("dk"), py::arg("dv"), py::arg("scale"));
    m.def("pack_mask", &pack_mask, "Pack a bool mask into uint32 words (returned as int32)",
          py::arg("mask"));
    m.def("version", []() { return sma_version(); });
}

// Python module `sparse_attn_cuda`: a thin pybind11 shim over the C ABI of libsma_hip.so.
//
// It keeps the module name and the two Python-visible signatures of the reference binding
// (csrc/binding.cpp:9-18 `forward`, csrc/binding.cpp:49 `pack_mask`, registered at
// csrc/binding.cpp:68-71) so that python/sparse_attention.py can stay as it is:
//
//   forward(q, k, v, mask_packed, out, lse, scale, is_training, tile_map=None) -> None
//   pack_mask(mask) -> int32 Tensor [B, H, N, ceil(N/32)]
//   tile_map(mask_packed) -> int32 Tensor [B, H, ceil(N/64), 2, ceil(ceil(N/64)/32)]   (not in the
//       reference: which 64 x 64 blocks of the mask hold a set bit / nothing but set bits; passed to
//       `forward` as tile_map, key tiles without a set bit are neither loaded nor computed)
//   backward(dout, q, k, v, out, lse, mask_packed, dq, dk, dv, scale, tile_map=None) -> None   (called by the
//       reference's Python API, python/sparse_attention.py:91-94, but absent from its binding)
//   forward_bool_mask(q, k, v, mask, out, lse, scale, is_training, packed_out=None, map_out=None) -> None   (not in
//       the reference: `forward` with the boolean mask itself in place of the packed one, one launch
//       instead of pack_mask + forward; `packed_out`, if given, receives what pack_mask would
//       return and `map_out` what tile_map would return for it; `bool_mask_supported(q, k, v, mask)`
//       says whether it applies)
//
// Differences, all on the safe side: `lse` may be None (the reference's own inference wrapper
// passes None, python/sparse_attention.py:170-171); every tensor argument is checked (device,
// dtype, shape, layout, head_dim 32, 64 or 128) instead of only `q`; launches go to the current HIP
// stream of q's device under a device guard; a failed launch raises RuntimeError.
// q, k, v, out and the gradients need not be contiguous: any view whose last dimension is
// contiguous and whose other strides are multiples of 8 elements is passed on with its strides
// (the reference reserves such strides, csrc/sparse_attention.h:30-33, and ignores them), and
// mask_packed may be [1|B, 1|H, N, ceil(N/32)]: a size of 1 shares the mask between batch
// entries / heads.
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

// Descriptor of a [B,H,N,D] tensor for the strided C entry points.  Extents of size 1 get stride 0
// (PyTorch leaves their strides arbitrary).
sma_tensor rows_of(const torch::Tensor &t, const char *name)
{
    if (t.numel() == 0) return sma_tensor{t.data_ptr(), 0, 0, 0};     // nothing will be read or written
    TORCH_CHECK(t.stride(3) == 1 || t.size(3) == 1, name, ": the last dimension must be contiguous");
    sma_tensor d;
    d.data = t.data_ptr();
    d.stride_b = t.size(0) == 1 ? 0 : t.stride(0);
    d.stride_h = t.size(1) == 1 ? 0 : t.stride(1);
    d.stride_n = t.size(2) == 1 ? 0 : t.stride(2);
    TORCH_CHECK(((d.stride_b | d.stride_h | d.stride_n) & 7) == 0 && d.stride_b >= 0 && d.stride_h >= 0 &&
                    d.stride_n >= 0,
                name, ": strides must be non-negative multiples of 8 elements (call .contiguous())");
    return d;
}

// Checks mask_packed ([1|B, 1|H, N, nw] int32, contiguous) and returns its word strides (0 = shared).
void mask_strides(const torch::Tensor &mp, const torch::Tensor &q, int64_t *sb, int64_t *sh)
{
    const int64_t B = q.size(0), H = q.size(1), N = q.size(2), nw = (N + 31) / 32;
    TORCH_CHECK(mp.device() == q.device(), "mask_packed must be on q's device");
    TORCH_CHECK(mp.scalar_type() == at::kInt, "mask_packed must be int32");
    TORCH_CHECK(mp.dim() == 4 && (mp.size(0) == B || mp.size(0) == 1) && (mp.size(1) == H || mp.size(1) == 1) &&
                    mp.size(2) == N && mp.size(3) == nw,
                "mask_packed must be [B or 1, H or 1, N, ceil(N/32)]");
    TORCH_CHECK(mp.is_contiguous(), "mask_packed must be contiguous");
    *sb = mp.size(0) == 1 ? 0 : mp.size(1) * N * nw;
    *sh = mp.size(1) == 1 ? 0 : N * nw;
}

// The optional tile map of mask_packed ([Bm, Hm, T, 2, ceil(T/32)] int32, T = ceil(N/64)), checked; nullptr if absent.
const uint32_t *map_pointer(const c10::optional<torch::Tensor> &tile_map, const torch::Tensor &mask_packed,
                            const torch::Tensor &q)
{
    if (!tile_map.has_value() || !tile_map->defined()) return nullptr;
    const torch::Tensor &m = *tile_map;
    const int64_t T = (q.size(2) + 63) / 64;
    TORCH_CHECK(m.device() == q.device() && m.scalar_type() == at::kInt && m.dim() == 5 &&
                    m.size(0) == mask_packed.size(0) && m.size(1) == mask_packed.size(1) && m.size(2) == T &&
                    m.size(3) == 2 && m.size(4) == (T + 31) / 32 && m.is_contiguous(),
                "tile_map must be the contiguous int32 result of tile_map(mask_packed)");
    return reinterpret_cast<const uint32_t *>(m.data_ptr<int32_t>());
}

void forward(const torch::Tensor &q, const torch::Tensor &k, const torch::Tensor &v,
             const torch::Tensor &mask_packed, torch::Tensor out,
             const c10::optional<torch::Tensor> &lse, double scale, bool is_training,
             const c10::optional<torch::Tensor> &tile_map)
{
    TORCH_CHECK(q.is_cuda(), "q must be a GPU tensor");
    TORCH_CHECK(q.dim() == 4, "q must be 4D [B, H, N, D]");
    const auto dt = q.scalar_type();
    TORCH_CHECK(dt == at::kHalf || dt == at::kBFloat16, "Unsupported dtype, need BF16 or FP16");
    const int64_t B = q.size(0), H = q.size(1), N = q.size(2), D = q.size(3);
    TORCH_CHECK(D == 32 || D == 64 || D == 128, "head_dim must be 32, 64 or 128, got ", D);
    for (const torch::Tensor *t : {&k, &v, static_cast<const torch::Tensor *>(&out)}) {
        TORCH_CHECK(t->device() == q.device(), "q, k, v, out must be on the same device");
        TORCH_CHECK(t->scalar_type() == dt, "q, k, v, out must have the same dtype");
        TORCH_CHECK(t->sizes() == q.sizes(), "q, k, v, out must have the same shape");
    }
    const sma_tensor tq = rows_of(q, "q"), tk = rows_of(k, "k"), tv = rows_of(v, "v"), to = rows_of(out, "out");
    int64_t msb = 0, msh = 0;
    mask_strides(mask_packed, q, &msb, &msh);
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
    const uint32_t *map_ptr = map_pointer(tile_map, mask_packed, q);

    const c10::DeviceGuard guard(q.device());
    hipStream_t stream = c10::hip::getCurrentHIPStream(q.device().index()).stream();
    const int st = sma_attn_fwd_map_strided(&tq, &tk, &tv,
                                            reinterpret_cast<const uint32_t *>(mask_packed.data_ptr<int32_t>()),
                                            msb, msh, map_ptr, &to, lse_ptr, (int)B, (int)H, (int)N, (int)D,
                                            (float)scale, dt == at::kBFloat16 ? SMA_DTYPE_BF16 : SMA_DTYPE_F16,
                                            stream);
    check_status(st, "sma_attn_fwd_map_strided");
}

// Limits of sma_attn_fwd_bool_mask, so that callers can choose between it and pack_mask + forward
// without provoking an error: q, k, v with contiguous rows and strides that are multiples of 8
// elements, head dim 32, 64 or 128, 16 <= N < 46341, a contiguous bool mask [1|B, 1|H, N, N].
bool bool_mask_supported(const torch::Tensor &q, const torch::Tensor &k, const torch::Tensor &v,
                         const torch::Tensor &mask)
{
    if (!q.is_cuda() || q.dim() != 4 || mask.dim() != 4) return false;
    const int64_t B = q.size(0), H = q.size(1), N = q.size(2), D = q.size(3);
    if (!(D == 32 || D == 64 || D == 128) || N < 16 || N * N >= (int64_t(1) << 31)) return false;
    // q, k, v as the strided entry points take them: rows contiguous, other strides multiples of 8
    // elements, 16-byte aligned storage
    for (const torch::Tensor *t : {&q, &k, &v}) {
        if (t->dim() != 4 || t->sizes() != q.sizes() || (t->stride(3) != 1 && t->size(3) != 1)) return false;
        if (reinterpret_cast<uintptr_t>(t->data_ptr()) % 16 != 0) return false;
        for (int d = 0; d < 3; ++d)
            if (t->size(d) > 1 && (t->stride(d) < 0 || t->stride(d) % 8 != 0)) return false;
    }
    if (mask.scalar_type() != at::kBool || !mask.is_contiguous() || mask.device() != q.device()) return false;
    if (!((mask.size(0) == B || mask.size(0) == 1) && (mask.size(1) == H || mask.size(1) == 1) &&
          mask.size(2) == N && mask.size(3) == N))
        return false;
    // the kernel copies mask rows from whatever byte address they start at: the library checks once
    // per device that such copies are served (always, under ROCm); where not, pack_mask + forward
    const c10::DeviceGuard guard(q.device());
    return sma_device_check(c10::hip::getCurrentHIPStream(q.device().index()).stream()) == SMA_OK;
}

void forward_bool_mask(const torch::Tensor &q, const torch::Tensor &k, const torch::Tensor &v,
                       const torch::Tensor &mask, torch::Tensor out,
                       const c10::optional<torch::Tensor> &lse, double scale, bool is_training,
                       const c10::optional<torch::Tensor> &packed_out,
                       const c10::optional<torch::Tensor> &map_out)
{
    TORCH_CHECK(q.is_cuda(), "q must be a GPU tensor");
    TORCH_CHECK(q.dim() == 4, "q must be 4D [B, H, N, D]");
    const auto dt = q.scalar_type();
    TORCH_CHECK(dt == at::kHalf || dt == at::kBFloat16, "Unsupported dtype, need BF16 or FP16");
    TORCH_CHECK(bool_mask_supported(q, k, v, mask),
                "forward_bool_mask needs q, k, v with contiguous rows (strides multiples of 8 elements), head_dim "
                "32, 64 or 128, N >= 16 and a contiguous bool mask [B or 1, H or 1, N, N]; use pack_mask + forward otherwise");
    const int64_t B = q.size(0), H = q.size(1), N = q.size(2), D = q.size(3);
    for (const torch::Tensor *t : {&k, &v, static_cast<const torch::Tensor *>(&out)}) {
        TORCH_CHECK(t->device() == q.device(), "q, k, v, out must be on the same device");
        TORCH_CHECK(t->scalar_type() == dt, "q, k, v, out must have the same dtype");
        TORCH_CHECK(t->sizes() == q.sizes(), "q, k, v, out must have the same shape");
    }
    const sma_tensor tq = rows_of(q, "q"), tk = rows_of(k, "k"), tv = rows_of(v, "v"), to = rows_of(out, "out");
    float *lse_ptr = nullptr;
    if (is_training) {
        TORCH_CHECK(lse.has_value() && lse->defined(), "is_training=True needs an lse tensor");
        TORCH_CHECK(lse->device() == q.device() && lse->scalar_type() == at::kFloat &&
                        lse->dim() == 3 && lse->size(0) == B && lse->size(1) == H &&
                        lse->size(2) == N && lse->is_contiguous(),
                    "lse must be a contiguous float32 [B, H, N] tensor on q's device");
        lse_ptr = lse->data_ptr<float>();
    }
    uint32_t *packed_ptr = nullptr;
    if (packed_out.has_value() && packed_out->defined()) {
        const torch::Tensor &p = *packed_out;
        TORCH_CHECK(p.device() == q.device() && p.scalar_type() == at::kInt && p.dim() == 4 &&
                        p.size(0) == mask.size(0) && p.size(1) == mask.size(1) && p.size(2) == N &&
                        p.size(3) == (N + 31) / 32 && p.is_contiguous(),
                    "packed_out must be a contiguous int32 [mask.size(0), mask.size(1), N, ceil(N/32)] tensor on q's device");
        packed_ptr = reinterpret_cast<uint32_t *>(p.data_ptr<int32_t>());
    }
    uint32_t *map_ptr = nullptr;
    if (map_out.has_value() && map_out->defined()) {
        const torch::Tensor &m = *map_out;
        const int64_t T = (N + 63) / 64;
        TORCH_CHECK(m.device() == q.device() && m.scalar_type() == at::kInt && m.dim() == 5 &&
                        m.size(0) == mask.size(0) && m.size(1) == mask.size(1) && m.size(2) == T &&
                        m.size(3) == 2 && m.size(4) == (T + 31) / 32 && m.is_contiguous(),
                    "map_out must be a contiguous int32 [mask.size(0), mask.size(1), T, 2, ceil(T/32)] tensor "
                    "on q's device, T = ceil(N/64)");
        map_ptr = reinterpret_cast<uint32_t *>(m.data_ptr<int32_t>());
    }
    const int64_t msb = mask.size(0) == 1 ? 0 : mask.size(1) * N * N;
    const int64_t msh = mask.size(1) == 1 ? 0 : N * N;
    const c10::DeviceGuard guard(q.device());
    hipStream_t stream = c10::hip::getCurrentHIPStream(q.device().index()).stream();
    const int st = sma_attn_fwd_bool_mask_strided(&tq, &tk, &tv,
                                                  reinterpret_cast<const uint8_t *>(mask.data_ptr<bool>()), msb, msh,
                                                  &to, lse_ptr, packed_ptr, map_ptr, (int)B, (int)H, (int)N,
                                                  (int)D, (float)scale,
                                                  dt == at::kBFloat16 ? SMA_DTYPE_BF16 : SMA_DTYPE_F16, stream);
    check_status(st, "sma_attn_fwd_bool_mask_strided");
}

// backward(dout, q, k, v, out, lse, mask_packed, dq, dk, dv, scale) -> None, the call the
// reference's autograd function makes (python/sparse_attention.py:91-94) to a function its
// binding never had.  dq, dk, dv are overwritten (not accumulated into).
void backward(const torch::Tensor &dout, const torch::Tensor &q, const torch::Tensor &k,
              const torch::Tensor &v, const torch::Tensor &out, const torch::Tensor &lse,
              const torch::Tensor &mask_packed, torch::Tensor dq, torch::Tensor dk,
              torch::Tensor dv, double scale, const c10::optional<torch::Tensor> &tile_map)
{
    TORCH_CHECK(q.is_cuda(), "q must be a GPU tensor");
    TORCH_CHECK(q.dim() == 4, "q must be 4D [B, H, N, D]");
    const auto dt = q.scalar_type();
    TORCH_CHECK(dt == at::kHalf || dt == at::kBFloat16, "Unsupported dtype, need BF16 or FP16");
    const int64_t B = q.size(0), H = q.size(1), N = q.size(2), D = q.size(3);
    TORCH_CHECK(D == 32 || D == 64 || D == 128, "head_dim must be 32, 64 or 128, got ", D);
    const torch::Tensor *all[8] = {&dout, &q, &k, &v, &out, &dq, &dk, &dv};
    const char *names[8] = {"dout", "q", "k", "v", "out", "dq", "dk", "dv"};
    sma_tensor d[8];
    for (int i = 0; i < 8; ++i) {
        const torch::Tensor *t = all[i];
        TORCH_CHECK(t->device() == q.device(), "dout, q, k, v, out, dq, dk, dv must be on the same device");
        TORCH_CHECK(t->scalar_type() == dt, "dout, q, k, v, out, dq, dk, dv must have the same dtype");
        TORCH_CHECK(t->sizes() == q.sizes(), "dout, q, k, v, out, dq, dk, dv must have the same shape");
        d[i] = rows_of(*t, names[i]);
    }
    int64_t msb = 0, msh = 0;
    mask_strides(mask_packed, q, &msb, &msh);
    TORCH_CHECK(lse.device() == q.device() && lse.scalar_type() == at::kFloat && lse.dim() == 3 &&
                    lse.size(0) == B && lse.size(1) == H && lse.size(2) == N && lse.is_contiguous(),
                "lse must be a contiguous float32 [B, H, N] tensor on q's device");
    TORCH_CHECK(B <= INT32_MAX && H <= INT32_MAX && N <= INT32_MAX, "extent too large");

    const uint32_t *map_ptr = map_pointer(tile_map, mask_packed, q);

    const c10::DeviceGuard guard(q.device());
    torch::Tensor delta = torch::empty({B, H, N}, lse.options());      // workspace of the C entry point
    hipStream_t stream = c10::hip::getCurrentHIPStream(q.device().index()).stream();
    const int st = sma_attn_bwd_map_strided(&d[0], &d[1], &d[2], &d[3], &d[4], lse.data_ptr<float>(),
                                            reinterpret_cast<const uint32_t *>(mask_packed.data_ptr<int32_t>()),
                                            msb, msh, map_ptr, &d[5], &d[6], &d[7], delta.data_ptr<float>(), (int)B,
                                            (int)H, (int)N, (int)D, (float)scale,
                                            dt == at::kBFloat16 ? SMA_DTYPE_BF16 : SMA_DTYPE_F16, stream);
    check_status(st, "sma_attn_bwd_map_strided");
}

torch::Tensor pack_mask(const torch::Tensor &mask)
{
    TORCH_CHECK(mask.is_cuda(), "mask must be a GPU tensor");
    TORCH_CHECK(mask.dim() == 4, "mask must be 4D [B, H, N, N]");
    TORCH_CHECK(mask.scalar_type() == at::kBool, "mask must be bool");
    TORCH_CHECK(mask.size(2) == mask.size(3), "mask must be [B, H, N, N]");
    // a mask shared between batch entries / heads is given as [1 or B, 1 or H, N, N] and packed as it is
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

// tile_map(mask_packed): [Bm, Hm, N, ceil(N/32)] int32 -> [Bm, Hm, T, 2, ceil(T/32)] int32, T = ceil(N/64).
torch::Tensor tile_map(const torch::Tensor &mask_packed)
{
    TORCH_CHECK(mask_packed.is_cuda(), "mask_packed must be a GPU tensor");
    TORCH_CHECK(mask_packed.scalar_type() == at::kInt && mask_packed.dim() == 4 && mask_packed.is_contiguous(),
                "mask_packed must be a contiguous int32 [B, H, N, ceil(N/32)] tensor");
    const int64_t B = mask_packed.size(0), H = mask_packed.size(1), N = mask_packed.size(2);
    TORCH_CHECK(mask_packed.size(3) == (N + 31) / 32, "mask_packed must be [B, H, N, ceil(N/32)]");
    TORCH_CHECK(B <= INT32_MAX && H <= INT32_MAX && N <= 131072, "extent too large");
    const int64_t T = (N + 63) / 64;
    const c10::DeviceGuard guard(mask_packed.device());
    torch::Tensor map = torch::empty({B, H, T, 2, (T + 31) / 32}, mask_packed.options());    // every word is written
    hipStream_t stream = c10::hip::getCurrentHIPStream(mask_packed.device().index()).stream();
    const int st = sma_tile_map(reinterpret_cast<const uint32_t *>(mask_packed.data_ptr<int32_t>()),
                                reinterpret_cast<uint32_t *>(map.data_ptr<int32_t>()), (int)B, (int)H, (int)N, stream);
    check_status(st, "sma_tile_map");
    return map;
}

}  // namespace

PYBIND11_MODULE(sparse_attn_cuda, m)
{
    m.doc() = "sparse-mask attention for MI355X (gfx950): pybind shim over libsma_hip.so";
    m.def("forward", &forward, "Sparse-mask attention forward", py::arg("q"), py::arg("k"),
          py::arg("v"), py::arg("mask_packed"), py::arg("out"), py::arg("lse"), py::arg("scale"),
          py::arg("is_training"), py::arg("tile_map") = py::none());
    m.def("tile_map", &tile_map,
          "Which 64 x 64 blocks of a packed mask hold a set bit / only set bits (pass to forward as tile_map)",
          py::arg("mask_packed"));
    m.def("backward", &backward, "Sparse-mask attention backward (dq, dk, dv are overwritten)",
          py::arg("dout"), py::arg("q"), py::arg("k"), py::arg("v"), py::arg("out"), py::arg("lse"),
          py::arg("mask_packed"), py::arg("dq"), py::arg("dk"), py::arg("dv"), py::arg("scale"),
          py::arg("tile_map") = py::none());
    m.def("forward_bool_mask", &forward_bool_mask,
          "Sparse-mask attention forward straight from the bool mask (one launch; see bool_mask_supported)",
          py::arg("q"), py::arg("k"), py::arg("v"), py::arg("mask"), py::arg("out"), py::arg("lse"),
          py::arg("scale"), py::arg("is_training"), py::arg("packed_out") = py::none(),
          py::arg("map_out") = py::none());
    m.def("bool_mask_supported", &bool_mask_supported,
          "Whether forward_bool_mask applies to these tensors (else use pack_mask + forward)", py::arg("q"),
          py::arg("k"), py::arg("v"), py::arg("mask"));
    m.def("pack_mask", &pack_mask, "Pack a bool mask into uint32 words (returned as int32)",
          py::arg("mask"));
    m.def("version", []() { return sma_version(); });
}

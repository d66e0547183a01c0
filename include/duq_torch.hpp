// duq_torch.hpp - header-only libtorch (C++) twin of the Linear4bit path over the C ABI in
// duq_hip.h, with the class and function names of the reference's C++ API:
//   PackedQuantizedTensor, PackedDoubleQuantizedTensor, Quantizer4bit, DeQuantizer4bit, sym_quant,
//   sym_dual_quant, sym_dequant, sym_dual_dequant, pack_i4          include/quant_tensor.h:11-90, src/module/quant_tensor.cu
//   Linear4bit, Linear4bitDUQ          include/linear.h:31-60,    src/module/linear.cu:83-281
// Tensors live on a ROCm device ("cuda" device type in PyTorch-ROCm); every call launches on
// torch's current HIP stream.  Argument errors raise c10::Error through TORCH_CHECK like the
// reference's torch::check* calls; a non-zero status of the C ABI raises too.
//
// Build: hipcc / g++ with the libtorch include paths, -DUSE_ROCM -D__HIP_PLATFORM_AMD__, link
// libduq_hip.so, libtorch, libc10, libc10_hip.
#pragma once

#include <torch/torch.h>

#include <c10/hip/HIPStream.h>

#include <tuple>
#include <utility>
#include <vector>

#include "duq_hip.h"

namespace duq {

inline duq_stream_t current_stream(const torch::Tensor &t)
{
    return static_cast<duq_stream_t>(c10::hip::getCurrentHIPStream(t.device().index()).stream());
}

inline void check_status(int status, const char *what) { TORCH_CHECK(status == DUQ_OK, what, ": ", duq_status_string(status)); }

inline void check_device_tensor(const torch::Tensor &t, const char *what, const char *name)
{
    TORCH_CHECK(t.is_contiguous(), what, ": expected ", name, " to be contiguous");
    TORCH_CHECK(t.is_cuda(), what, ": expected ", name, " to be on a GPU device");
}

inline const duq_half *half_ptr(const torch::Tensor &t)
{
    TORCH_CHECK(t.scalar_type() == torch::kFloat16, "expected a float16 tensor");  // bf16 storage is rejected
    return reinterpret_cast<const duq_half *>(t.data_ptr());
}

// [..., K] -> ([rows, K], leading sizes)
inline std::pair<torch::Tensor, std::vector<int64_t>> flatten_last_dim_and_return_shape(const torch::Tensor &x)
{
    std::vector<int64_t> lead(x.sizes().begin(), x.sizes().end() - 1);
    return {x.view({-1, x.size(-1)}), lead};
}

// ---- quantized activation (include/quant_tensor.h:11-27)
// A few rows (decode) may arrive *deferred* from Quantizer4bit: the object then holds the binary16 rows
// (`source_x`) and the quantizer's settings, quantized_x / scale are undefined, and a Linear4bit / Linear4bitDUQ
// that can run quantizer + GEMM + dequant as one launch consumes the rows directly.  Anything else calls
// materialize() first (one quantizer launch, the same bits); Quantizer4bit(clip, qmax, shadow, 0) never defers.
class PackedQuantizedTensor {
public:
    torch::Tensor quantized_x;
    torch::Tensor scale;
    // not in the reference: the same codes as 6-bit floats [..., 3K/4] for the 6-bit float matrix path
    // (Quantizer4bit with shadow = true); undefined otherwise
    torch::Tensor shadow_x;
    // not in the reference: the deferred form (see above); undefined otherwise
    torch::Tensor source_x;
    float clip = 1.0f;
    int qmax = DUQ_QMAX_SYM_DEVICE;

    PackedQuantizedTensor(torch::Tensor quantized_x, torch::Tensor scale, torch::Tensor shadow_x = torch::Tensor())
        : quantized_x(std::move(quantized_x)), scale(std::move(scale)), shadow_x(std::move(shadow_x)) {}

    static PackedQuantizedTensor deferred(torch::Tensor x, float clip, int qmax)
    {
        PackedQuantizedTensor p{torch::Tensor(), torch::Tensor()};
        p.packed_sizes_.assign(x.sizes().begin(), x.sizes().end());
        p.packed_sizes_.back() /= 2;
        p.source_x = std::move(x);
        p.clip = clip;
        p.qmax = qmax;
        return p;
    }
    bool is_deferred() const { return source_x.defined(); }

    // Run the quantizer now (no-op unless deferred): quantized_x [..., K/2] and scale [..., 1] as Quantizer4bit
    // writes them for larger inputs.
    PackedQuantizedTensor &materialize()
    {
        if (!source_x.defined()) return *this;
        const torch::Tensor &x = source_x;
        const uint32_t cols = x.size(-1), rows = cols ? x.numel() / cols : 0;
        std::vector<int64_t> qshape(x.sizes().begin(), x.sizes().end()), sshape = qshape;
        qshape.back() = cols / 2;
        sshape.back() = 1;
        quantized_x = torch::empty(qshape, torch::dtype(torch::kUInt8).device(x.device()));
        scale = torch::empty(sshape, torch::dtype(torch::kHalf).device(x.device()));
        const int st = duq_quantize_rows_sym(reinterpret_cast<const duq_half *>(x.data_ptr()), rows, cols, clip, qmax,
                                             quantized_x.data_ptr<uint8_t>(), reinterpret_cast<duq_half *>(scale.data_ptr()),
                                             static_cast<duq_stream_t>(c10::hip::getCurrentHIPStream(x.device().index()).stream()));
        TORCH_CHECK(st == DUQ_OK, "PackedQuantizedTensor::materialize: ", duq_status_string(st));
        source_x = torch::Tensor();
        return *this;
    }

    torch::IntArrayRef sizes() const { return source_x.defined() ? torch::IntArrayRef(packed_sizes_) : quantized_x.sizes(); }
    torch::Device device() const { return source_x.defined() ? source_x.device() : quantized_x.device(); }

private:
    std::vector<int64_t> packed_sizes_;
};

// quantized activation with two scales: columns < 10 and the rest (include/quant_tensor.h:29-45)
class PackedDoubleQuantizedTensor {
public:
    torch::Tensor quantized_x;
    torch::Tensor scale_1;
    torch::Tensor scale_2;
    PackedDoubleQuantizedTensor(torch::Tensor quantized_x, torch::Tensor scale_1, torch::Tensor scale_2)
        : quantized_x(std::move(quantized_x)), scale_1(std::move(scale_1)), scale_2(std::move(scale_2)) {}
    torch::IntArrayRef sizes() const { return quantized_x.sizes(); }
    torch::Device device() const { return quantized_x.device(); }
};

// ---- tensor-level ops (src/module/quant_tensor.cu:11-148)
inline torch::Tensor sym_quant(const torch::Tensor &x, const torch::Tensor &scale, int qmax = DUQ_QMAX_SYM_DEVICE)
{
    check_device_tensor(x, "sym_quant", "x");
    check_device_tensor(scale, "sym_quant", "scale");
    TORCH_CHECK(x.dim() == 2 && scale.size(0) == x.size(0), "sym_quant: expected scale to have size ", x.size(0), " at dimension 0");
    const uint32_t rows = x.size(0), cols = x.size(1), cd = (cols + 1) / 2;
    auto q = torch::empty({rows, cd}, torch::dtype(torch::kUInt8).device(x.device()));
    check_status(duq_sym_quant_host_qmax(half_ptr(x), half_ptr(scale), rows, cols, cd, qmax, q.data_ptr<uint8_t>(),
                                         current_stream(x)),
                 "sym_quant");
    return q;
}

// columns < 10 of every row use scale_1, the others scale_2 (src/module/quant_tensor.cu:31-57)
inline torch::Tensor sym_dual_quant(const torch::Tensor &x, const torch::Tensor &scale_1, const torch::Tensor &scale_2)
{
    check_device_tensor(x, "sym_dual_quant", "x");
    check_device_tensor(scale_1, "sym_dual_quant", "scale_1");
    check_device_tensor(scale_2, "sym_dual_quant", "scale_2");
    TORCH_CHECK(x.dim() == 2 && scale_1.size(0) == x.size(0) && scale_2.size(0) == x.size(0),
                "sym_dual_quant: expected both scales to have size ", x.size(0), " at dimension 0");
    const uint32_t rows = x.size(0), cols = x.size(1), cd = (cols + 1) / 2;
    auto q = torch::empty({rows, cd}, torch::dtype(torch::kUInt8).device(x.device()));
    check_status(duq_sym_dual_quant_host(half_ptr(x), half_ptr(scale_1), half_ptr(scale_2), rows, cols, cd,
                                         q.data_ptr<uint8_t>(), current_stream(x)),
                 "sym_dual_quant");
    return q;
}

inline torch::Tensor sym_dequant(const torch::Tensor &q, const torch::Tensor &scale_row, const torch::Tensor &scale_col, int bits)
{
    check_device_tensor(q, "sym_dequant", "q");
    check_device_tensor(scale_row, "sym_dequant", "scale_row");
    check_device_tensor(scale_col, "sym_dequant", "scale_col");
    TORCH_CHECK(bits == 32, "Unsupported data type");  // src/module/quant_tensor.cu:93-96
    TORCH_CHECK(q.scalar_type() == torch::kInt32 && q.dim() == 2, "sym_dequant: q must be int32 [rows, cols]");
    const uint32_t rows = q.size(0), cols = q.size(1);
    TORCH_CHECK(scale_row.size(0) == rows && scale_col.size(0) == cols, "sym_dequant: scale sizes do not match q");
    auto x = torch::empty(q.sizes(), torch::dtype(torch::kHalf).device(q.device()));
    check_status(duq_sym_dequant_host(q.data_ptr<int32_t>(), half_ptr(scale_row), half_ptr(scale_col), rows, cols,
                                      reinterpret_cast<duq_half *>(x.data_ptr()), current_stream(q)),
                 "sym_dequant");
    return x;
}

inline torch::Tensor sym_dual_dequant(const torch::Tensor &q, const torch::Tensor &scale_row, const torch::Tensor &scale_col_1,
                                      const torch::Tensor &scale_col_2, int bits)
{
    check_device_tensor(q, "sym_dual_dequant", "q");
    TORCH_CHECK(bits == 32, "Unsupported data type");
    TORCH_CHECK(q.scalar_type() == torch::kInt32 && q.dim() == 2, "sym_dual_dequant: q must be int32 [rows, cols]");
    const uint32_t rows = q.size(0), cols = q.size(1);
    TORCH_CHECK(scale_row.size(0) == rows && scale_col_1.size(0) == cols && scale_col_2.size(0) == cols,
                "sym_dual_dequant: scale sizes do not match q");
    auto x = torch::empty(q.sizes(), torch::dtype(torch::kHalf).device(q.device()));
    check_status(duq_sym_dual_dequant_host(q.data_ptr<int32_t>(), half_ptr(scale_row), half_ptr(scale_col_1),
                                           half_ptr(scale_col_2), rows, cols, reinterpret_cast<duq_half *>(x.data_ptr()),
                                           current_stream(q)),
                 "sym_dual_dequant");
    return x;
}

// int4Unpack(A) @ int4Unpack(B)^T -> int32 (src/export/bindings.cpp:10-26)
inline torch::Tensor matmul(const torch::Tensor &A, const torch::Tensor &B)
{
    check_device_tensor(A, "matmul", "A");
    check_device_tensor(B, "matmul", "B");
    TORCH_CHECK(A.dim() == 2 && B.dim() == 2 && A.size(1) == B.size(1), "matmul: packed K differs");
    const uint32_t M = A.size(0), N = B.size(0), K = A.size(1) * 2;
    auto C = torch::empty({M, N}, torch::dtype(torch::kInt32).device(A.device()));
    check_status(duq_matmul_host_4bit(A.data_ptr<uint8_t>(), B.data_ptr<uint8_t>(), M, N, K, C.data_ptr<int32_t>(), current_stream(A)),
                 "matmul");
    return C;
}

// signed integer tensor [rows, K] with values in [-8, 7] -> uint8 [rows, K/2] (quant_tensor.cu:197-206)
inline torch::Tensor pack_i4(const torch::Tensor &q)
{
    TORCH_CHECK(q.dim() == 2 && q.size(1) % 2 == 0, "pack_i4: expected [rows, even K]");
    TORCH_CHECK(torch::all(q.ge(-8).logical_and(q.le(7))).item<bool>(), "pack_i4: value outside the int4 range");
    auto codes = torch::where(q < 0, q + 16, q).to(torch::kUInt8);
    using torch::indexing::Slice;
    return codes.index({Slice(), Slice(0, torch::indexing::None, 2)}) |
           (codes.index({Slice(), Slice(1, torch::indexing::None, 2)}) * 16);
}

// ---- modules
// Per-token symmetric quantizer, one fused kernel (src/module/quant_tensor.cu:151-161)
class Quantizer4bit : public torch::nn::Module {
public:
    float input_clip_ratio;
    int qmax;
    bool shadow;  // also write the 6-bit float shadow (inputs whose width is a multiple of 128)
    // defer_rows > 0 (at most 1024 is useful): inputs of at most that many rows are handed on unquantized
    // (PackedQuantizedTensor::deferred) and the linear layer behind quantizes them inside its own library call (one
    // launch up to eight rows or sixteen short ones, the quantizer launch and the GEMM launch of one call above).  Off by default: the
    // fields quantized_x and scale of such a tensor are undefined until materialize(), and code written against the
    // reference reads them as plain members (test/test.cu:238-242).  A decode pipeline that only passes the tensor
    // on, torch::nn::Sequential(Quantizer4bit(clip, qmax, false, 64), Linear4bit) (test/pipeline.cu:107-110), turns it on.
    uint32_t defer_rows;
    explicit Quantizer4bit(float input_clip_ratio, int qmax = DUQ_QMAX_SYM_DEVICE, bool shadow = false, uint32_t defer_rows = 0)
        : input_clip_ratio(input_clip_ratio), qmax(qmax), shadow(shadow), defer_rows(defer_rows) {}
    PackedQuantizedTensor forward(torch::Tensor x)
    {
        x = x.contiguous();
        check_device_tensor(x, "Quantizer4bit::forward", "x");
        half_ptr(x);  // binary16 only (bf16 storage is rejected)
        auto [x2, lead] = flatten_last_dim_and_return_shape(x);
        const uint32_t rows = x2.size(0), cols = x2.size(1);
        TORCH_CHECK(cols % 32 == 0, "Quantizer4bit::forward: the last dimension must be a multiple of 32");
        if (!shadow && rows > 0 && rows <= defer_rows && cols % 64 == 0 && reinterpret_cast<uintptr_t>(x.data_ptr()) % 16 == 0)
            return PackedQuantizedTensor::deferred(x, input_clip_ratio, qmax);
        auto q = torch::empty({rows, cols / 2}, torch::dtype(torch::kUInt8).device(x.device()));
        auto s = torch::empty({rows, 1}, torch::dtype(torch::kHalf).device(x.device()));
        auto qshape = lead;
        qshape.push_back(cols / 2);
        auto sshape = lead;
        sshape.push_back(1);
        if (shadow && cols % 128 == 0) {
            auto b = torch::empty({rows, cols * 3 / 4}, torch::dtype(torch::kUInt8).device(x.device()));
            check_status(duq_quantize_rows_sym_bf6(half_ptr(x2), rows, cols, input_clip_ratio, qmax, q.data_ptr<uint8_t>(),
                                                   b.data_ptr<uint8_t>(), reinterpret_cast<duq_half *>(s.data_ptr()),
                                                   current_stream(x)),
                         "Quantizer4bit::forward");
            auto bshape = lead;
            bshape.push_back(cols * 3 / 4);
            return PackedQuantizedTensor(q.view(qshape), s.view(sshape), b.view(bshape));
        }
        check_status(duq_quantize_rows_sym(half_ptr(x2), rows, cols, input_clip_ratio, qmax, q.data_ptr<uint8_t>(),
                                           reinterpret_cast<duq_half *>(s.data_ptr()), current_stream(x)),
                     "Quantizer4bit::forward");
        return PackedQuantizedTensor(q.view(qshape), s.view(sshape));
    }
};

class DeQuantizer4bit : public torch::nn::Module {
public:
    uint32_t bits = 32;
    DeQuantizer4bit() {}
    explicit DeQuantizer4bit(uint32_t bits) : bits(bits) {}
    torch::Tensor forward(torch::Tensor &x, torch::Tensor &scale_x, torch::Tensor &weight_scale)
    {
        return sym_dequant(x, scale_x.view(-1), weight_scale, static_cast<int>(bits));
    }
};

namespace detail {
// E3M2 shadow of packed weights [N, K/2] -> [ceil(N/32)*32, 3K/4] (N % 16 == 0, K % 128 == 0)
inline torch::Tensor weight_shadow(const torch::Tensor &weight)
{
    check_device_tensor(weight, "weight_shadow", "weight");
    const uint32_t N = weight.size(0), K = weight.size(1) * 2;
    auto out = torch::empty({(N + 31) / 32 * 32, K * 3 / 4}, torch::dtype(torch::kUInt8).device(weight.device()));
    check_status(duq_weight_shadow_bf6(weight.data_ptr<uint8_t>(), N, K, out.data_ptr<uint8_t>(), current_stream(weight)),
                 "weight_shadow");
    return out;
}

// The 6-bit float matrix path is taken when both shadows exist and the problem has more rows than the integer
// decode kernel takes (64 of up to 8192 elements, 48 of up to 12288, 32 beyond; a shadow row holds 3/4 byte per
// element) and at least 32 output tiles of 64 x 256 (below, the integer kernels do better); same bits either way.
inline bool use_shadow(const PackedQuantizedTensor &input, const torch::Tensor &w_shadow, int64_t N)
{
    if (!input.shadow_x.defined() || !w_shadow.defined()) return false;
    const int64_t rows = input.shadow_x.numel() / input.shadow_x.size(-1);
    const int64_t K = input.shadow_x.size(-1) * 4 / 3;
    return rows > (K <= 8192 ? 64 : (K <= 12288 ? 48 : 32)) && ((rows + 63) / 64) * ((N + 255) / 256) >= 32;
}

inline torch::Tensor fused_forward_shadow(int mode, const PackedQuantizedTensor &input, const torch::Tensor &w_shadow,
                                          const torch::Tensor &s1, const torch::Tensor &s2, const torch::Tensor &bias)
{
    auto [A, lead] = flatten_last_dim_and_return_shape(input.shadow_x);
    check_device_tensor(A, "Linear4bit::forward", "shadow_x");
    TORCH_CHECK(A.device() == w_shadow.device(), "Linear4bit::forward: operands on different devices");
    TORCH_CHECK(w_shadow.size(1) == A.size(1), "Linear4bit::forward: shadow row length differs");
    const uint32_t M = A.size(0), N = s1.numel(), K = A.size(1) * 4 / 3;
    TORCH_CHECK(w_shadow.size(0) == (N + 31) / 32 * 32, "Linear4bit::forward: weight shadow rows do not match the scales");
    auto scale_row = input.scale.contiguous().view(-1);
    TORCH_CHECK(scale_row.size(0) == M, "Linear4bit::forward: one activation scale per token expected");
    auto y = torch::empty({M, N}, torch::dtype(torch::kHalf).device(A.device()));
    check_status(duq_linear4bit_forward_bf6(mode, A.data_ptr<uint8_t>(), half_ptr(scale_row), nullptr, nullptr,
                                            w_shadow.data_ptr<uint8_t>(), half_ptr(s1), nullptr,
                                            s2.defined() ? half_ptr(s2) : nullptr, nullptr, nullptr,
                                            bias.defined() ? half_ptr(bias) : nullptr, M, N, K,
                                            reinterpret_cast<duq_half *>(y.data_ptr()), current_stream(A)),
                 "Linear4bit::forward");
    lead.push_back(N);
    return y.view(lead);
}

// A deferred input of at most 1024 rows: quantizer + GEMM + dequant in one library call (ONE launch where the shape
// allows, else two with the codes and scales staged in a workspace allocated here); else an undefined tensor (the
// caller then materializes the input and takes the usual route).
inline torch::Tensor fused_decode(int mode, const PackedQuantizedTensor &input, const torch::Tensor &weight,
                                  const torch::Tensor &s1, const torch::Tensor &s2, const torch::Tensor &bias)
{
    const torch::Tensor &x = input.source_x;
    check_device_tensor(weight, "Linear4bit::forward", "B");
    TORCH_CHECK(x.device() == weight.device(), "Linear4bit::forward: operands on different devices");
    TORCH_CHECK(weight.size(1) * 2 == x.size(-1), "Linear4bit::forward: K differs");
    const uint32_t K = x.size(-1), M = x.numel() / K, N = weight.size(0);
    if (M > 1024) return torch::Tensor();
    const uint64_t ws_bytes = duq_quantize_linear4bit_workspace_bytes(M, N, K);
    torch::Tensor ws;
    if (ws_bytes) ws = torch::empty({(int64_t)ws_bytes}, torch::dtype(torch::kUInt8).device(x.device()));
    std::vector<int64_t> shape(x.sizes().begin(), x.sizes().end());
    shape.back() = N;
    auto y = torch::empty(shape, torch::dtype(torch::kHalf).device(x.device()));
    check_status(duq_quantize_linear4bit_forward(mode, half_ptr(x), input.clip, input.qmax, weight.data_ptr<uint8_t>(),
                                                 half_ptr(s1), s2.defined() ? half_ptr(s2) : nullptr,
                                                 bias.defined() ? half_ptr(bias) : nullptr, M, N, K,
                                                 reinterpret_cast<duq_half *>(y.data_ptr()), nullptr, nullptr,
                                                 ws_bytes ? ws.data_ptr() : nullptr, ws_bytes, current_stream(x)),
                 "Linear4bit::forward");
    return y;
}

inline torch::Tensor fused_forward(int mode, const PackedQuantizedTensor &input, const torch::Tensor &weight,
                                   const torch::Tensor &s1, const torch::Tensor &s2, const torch::Tensor &bias)
{
    const torch::Tensor &x = input.quantized_x;
    TORCH_CHECK(x.size(-1) % 32 == 0, "packed activation width must be a multiple of 32 bytes");  // linear.cu:115
    auto [A, lead] = flatten_last_dim_and_return_shape(x);
    check_device_tensor(A, "Linear4bit::forward", "A");
    check_device_tensor(weight, "Linear4bit::forward", "B");
    TORCH_CHECK(A.device() == weight.device(), "Linear4bit::forward: operands on different devices");
    const uint32_t M = A.size(0), N = weight.size(0), K = A.size(1) * 2;
    TORCH_CHECK(weight.size(1) == A.size(1), "Linear4bit::forward: packed K differs");
    auto scale_row = input.scale.contiguous().view(-1);
    TORCH_CHECK(scale_row.size(0) == M, "Linear4bit::forward: one activation scale per token expected");
    auto y = torch::empty({M, N}, torch::dtype(torch::kHalf).device(A.device()));
    check_status(duq_linear4bit_forward(mode, A.data_ptr<uint8_t>(), half_ptr(scale_row), nullptr, weight.data_ptr<uint8_t>(),
                                        half_ptr(s1), nullptr, s2.defined() ? half_ptr(s2) : nullptr, nullptr,
                                        bias.defined() ? half_ptr(bias) : nullptr, M, N, K,
                                        reinterpret_cast<duq_half *>(y.data_ptr()), current_stream(A)),
                 "Linear4bit::forward");
    lead.push_back(N);
    return y.view(lead);
}
}  // namespace detail

// Symmetric 4-bit linear layer (include/linear.h:31-45, src/module/linear.cu:83-176)
class Linear4bit : public torch::nn::Module {
public:
    torch::Tensor weight;        // uint8 [out, in/2]
    torch::Tensor weight_scale;  // fp16 [out, 1]
    torch::Tensor bias;          // fp16 [out] or undefined

    Linear4bit(uint32_t input_dim, uint32_t output_dim, bool use_bias, torch::Dtype dtype = torch::kFloat16)
    {
        weight = torch::zeros({output_dim, input_dim / 2}, torch::dtype(torch::kUInt8).device(torch::kCUDA));
        weight_scale = torch::zeros({output_dim, 1}, torch::dtype(dtype).device(torch::kCUDA));
        if (use_bias) bias = torch::zeros({output_dim}, torch::dtype(dtype).device(torch::kCUDA));
    }

    torch::Tensor weight_shadow;  // not in the reference: 6-bit float shadow of `weight`, see enable_fp6()

    // Build the 6-bit float shadow of the weights (3/4 byte per element more): large inputs quantized with
    // Quantizer4bit(..., shadow = true) then run on the 6-bit float matrix instruction, same bits, faster.
    // Call again after changing `weight`.
    Linear4bit &enable_fp6()
    {
        weight_shadow = detail::weight_shadow(weight);
        return *this;
    }

    torch::Tensor forward(PackedQuantizedTensor input)
    {
        if (input.is_deferred()) {  // a few rows straight from Quantizer4bit: quantized inside the GEMM launch
            auto y = detail::fused_decode(DUQ_EPI_SYM, input, weight, weight_scale.view(-1), torch::Tensor(), bias);
            if (y.defined()) return y;
            input.materialize();
        }
        if (detail::use_shadow(input, weight_shadow, weight.size(0)))
            return detail::fused_forward_shadow(DUQ_EPI_SYM, input, weight_shadow, weight_scale.view(-1), torch::Tensor(), bias);
        return detail::fused_forward(DUQ_EPI_SYM, input, weight, weight_scale.view(-1), torch::Tensor(), bias);
    }

    // round(W / weight_scales) packed to nibbles (src/module/linear.cu:161-176)
    static Linear4bit from_float(torch::nn::Linear &linear, torch::Tensor weight_scales)
    {
        auto w = linear->weight.detach().to(torch::kCUDA);
        Linear4bit out(w.size(1), w.size(0), linear->bias.defined(), w.scalar_type());
        TORCH_CHECK(weight_scales.dim() == 2 && weight_scales.size(0) == w.size(0) && weight_scales.size(1) == 1,
                    "weight_scales should have shape (out_features, 1)");
        out.weight_scale.copy_(weight_scales.to(w.scalar_type()));
        out.weight.copy_(pack_i4((w / weight_scales.to(w.device())).round().to(torch::kInt8)));
        if (linear->bias.defined()) out.bias.copy_(linear->bias.detach());
        return out;
    }
};

// Dual-uniform variant: output columns < 10 use weight_scale_1 (include/linear.h:48-60, linear.cu:178-281)
class Linear4bitDUQ : public torch::nn::Module {
public:
    torch::Tensor weight;
    torch::Tensor weight_scale_1;
    torch::Tensor weight_scale_2;
    torch::Tensor bias;

    Linear4bitDUQ(uint32_t input_dim, uint32_t output_dim, bool use_bias, torch::Dtype dtype = torch::kFloat16)
    {
        weight = torch::zeros({output_dim, input_dim / 2}, torch::dtype(torch::kUInt8).device(torch::kCUDA));
        weight_scale_1 = torch::zeros({output_dim, 1}, torch::dtype(dtype).device(torch::kCUDA));
        weight_scale_2 = torch::zeros({output_dim, 1}, torch::dtype(dtype).device(torch::kCUDA));
        if (use_bias) bias = torch::zeros({output_dim}, torch::dtype(dtype).device(torch::kCUDA));
    }

    torch::Tensor weight_shadow;  // see Linear4bit::enable_fp6()

    Linear4bitDUQ &enable_fp6()
    {
        weight_shadow = detail::weight_shadow(weight);
        return *this;
    }

    torch::Tensor forward(PackedQuantizedTensor input)
    {
        if (input.is_deferred()) {
            auto y = detail::fused_decode(DUQ_EPI_SYM_DUAL, input, weight, weight_scale_1.view(-1), weight_scale_2.view(-1), bias);
            if (y.defined()) return y;
            input.materialize();
        }
        if (detail::use_shadow(input, weight_shadow, weight.size(0)))
            return detail::fused_forward_shadow(DUQ_EPI_SYM_DUAL, input, weight_shadow, weight_scale_1.view(-1),
                                                weight_scale_2.view(-1), bias);
        return detail::fused_forward(DUQ_EPI_SYM_DUAL, input, weight, weight_scale_1.view(-1), weight_scale_2.view(-1), bias);
    }

    static Linear4bitDUQ from_float(torch::nn::Linear &linear, torch::Tensor weight_scales_1, torch::Tensor weight_scales_2)
    {
        auto w = linear->weight.detach().to(torch::kCUDA);
        Linear4bitDUQ out(w.size(1), w.size(0), linear->bias.defined(), w.scalar_type());
        out.weight_scale_1.copy_(weight_scales_1.to(w.scalar_type()));
        out.weight_scale_2.copy_(weight_scales_2.to(w.scalar_type()));
        const int64_t split = duq_get_dual_quant_col_k();
        auto left = (w.slice(1, 0, split) / weight_scales_1.to(w.device())).round();
        auto right = (w.slice(1, split) / weight_scales_2.to(w.device())).round();
        out.weight.copy_(pack_i4(torch::cat({left, right}, 1).to(torch::kInt8)));
        if (linear->bias.defined()) out.bias.copy_(linear->bias.detach());
        return out;
    }
};

}  // namespace duq

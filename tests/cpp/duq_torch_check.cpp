// Runs the libtorch classes of include/duq_torch.hpp on the current GPU and checks the fused
// Linear4bit / Linear4bitDUQ forwards against the three-step path (matmul, dequant, bias add)
// built from the same header, bit for bit.  Prints "OK <checksum>" and exits 0 on success.
//   duq_torch_check M K N            self-consistency at a given shape
//   duq_torch_check --fixture DIR    against the CPU oracle's expectations (raw arrays in DIR)
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#include "duq_torch.hpp"

static bool same_bits(const torch::Tensor &a, const torch::Tensor &b)
{
    return a.sizes() == b.sizes() && torch::equal(a.contiguous().view(torch::kInt16), b.contiguous().view(torch::kInt16));
}

// ---- fixture mode: inputs and expected outputs of the CPU oracle, handed over as raw arrays ----
static torch::Tensor read_raw(const std::string &dir, const char *name, torch::Dtype dtype, std::vector<int64_t> shape)
{
    auto t = torch::empty(shape, torch::dtype(dtype));
    const std::string path = dir + "/" + name + ".bin";
    FILE *f = std::fopen(path.c_str(), "rb");
    if (!f) { std::printf("FAIL cannot open %s\n", path.c_str()); std::exit(1); }
    const size_t want = (size_t)t.numel() * t.element_size();
    const size_t got = std::fread(t.data_ptr(), 1, want, f);
    std::fclose(f);
    if (got != want) { std::printf("FAIL %s holds %zu bytes, expected %zu\n", path.c_str(), got, want); std::exit(1); }
    return t;
}

// The classes against expectations that came from the CPU oracle (the arrays of tests/golden/linear4bit_small.npz
// written out one file each): quantizer codes and scales, from_float weight codes, and the forwards of both layers.
static int fixture_check(const std::string &dir)
{
    const int64_t M = 24, K = 256, N = 48;
    auto dev = torch::Device(torch::kCUDA, 0);
    auto H = torch::kHalf;
    auto x = read_raw(dir, "sym_x", H, {M, K}).to(dev);
    auto w_float = read_raw(dir, "sym_w_float", H, {N, K});
    auto bias = read_raw(dir, "bias", H, {N});
    auto sw = read_raw(dir, "sym_sw", H, {N, 1}).to(dev);

    torch::nn::Linear lin(torch::nn::LinearOptions(K, N).bias(true));
    lin->to(dev, H);
    {
        torch::NoGradGuard ng;
        lin->weight.copy_(w_float);
        lin->bias.copy_(bias);
    }
    for (int qmax : {6, 7}) {
        const std::string tag = "sym_q" + std::to_string(qmax);
        duq::Quantizer4bit quant(1.0f, qmax);
        auto p = quant.forward(x);
        if (!torch::equal(p.quantized_x.cpu(), read_raw(dir, (tag + "_qx").c_str(), torch::kUInt8, {M, K / 2}))) {
            std::printf("FAIL fixture quantizer codes qmax %d\n", qmax); return 1;
        }
        if (!same_bits(p.scale.cpu(), read_raw(dir, (tag + "_sx").c_str(), H, {M, 1}))) {
            std::printf("FAIL fixture quantizer scales qmax %d\n", qmax); return 1;
        }
        auto l = duq::Linear4bit::from_float(lin, sw);  // weight preparation on the device
        if (!torch::equal(l.weight.cpu(), read_raw(dir, "sym_w", torch::kUInt8, {N, K / 2}))) { std::puts("FAIL fixture from_float codes"); return 1; }
        auto acc = duq::matmul(p.quantized_x, l.weight);
        if (!torch::equal(acc.cpu(), read_raw(dir, (tag + "_acc").c_str(), torch::kInt32, {M, N}))) { std::puts("FAIL fixture accumulators"); return 1; }
        if (!same_bits(l.forward(p).cpu(), read_raw(dir, (tag + "_y").c_str(), H, {M, N}))) {
            std::printf("FAIL fixture Linear4bit forward qmax %d\n", qmax); return 1;
        }
        if (qmax == 6) {
            // the dual-uniform layer on the same codes with a second scale vector
            duq::Linear4bitDUQ d(K, N, true);
            d.weight.copy_(l.weight);
            d.weight_scale_1.copy_(sw);
            d.weight_scale_2.copy_(read_raw(dir, "dusq_sw2", H, {N, 1}));
            d.bias.copy_(bias);
            if (!same_bits(d.forward(p).cpu(), read_raw(dir, "dusq_y", H, {M, N}))) { std::puts("FAIL fixture Linear4bitDUQ forward"); return 1; }
            // and as its own from_float prepares it
            auto d2 = duq::Linear4bitDUQ::from_float(lin, read_raw(dir, "dusq_ff_s1", H, {N, 1}).to(dev),
                                                     read_raw(dir, "dusq_ff_s2", H, {N, 1}).to(dev));
            if (!torch::equal(d2.weight.cpu(), read_raw(dir, "dusq_ff_w", torch::kUInt8, {N, K / 2}))) { std::puts("FAIL fixture DUQ from_float codes"); return 1; }
            if (!same_bits(d2.forward(p).cpu(), read_raw(dir, "dusq_ff_y", H, {M, N}))) { std::puts("FAIL fixture DUQ from_float forward"); return 1; }
        }
    }
    torch::cuda::synchronize();
    std::puts("OK fixture");
    return 0;
}

int main(int argc, char **argv)
{
    if (argc > 2 && std::string(argv[1]) == "--fixture") return fixture_check(argv[2]);
    const int64_t M = argc > 1 ? atoll(argv[1]) : 48, K = argc > 2 ? atoll(argv[2]) : 256, N = argc > 3 ? atoll(argv[3]) : 192;
    torch::manual_seed(1234);
    auto dev = torch::Device(torch::kCUDA, 0);
    auto x = (torch::randn({3, M / 3, K}, torch::dtype(torch::kFloat32).device(dev)) * 1.5).to(torch::kHalf);

    torch::nn::Linear lin(torch::nn::LinearOptions(K, N).bias(true));
    lin->to(dev, torch::kHalf);
    auto w = lin->weight.detach();
    auto ws = (w.abs().amax(1, true).to(torch::kFloat32) / 7.0).to(torch::kHalf);

    duq::Quantizer4bit quant(1.0f);  // quantizes at once (the default; the decode hand-over is checked below)
    auto p = quant.forward(x);
    if (p.quantized_x.size(-1) != K / 2 || p.scale.size(-1) != 1 || p.scale.dim() != 3) { std::puts("FAIL quantizer shapes"); return 1; }

    // scale = h(h(max|x| / 7) * clip) with clip = 1, exact in float then rounded once
    auto want_scale = (x.abs().amax(-1, true).to(torch::kFloat32) / 7.0).to(torch::kHalf);
    if (!same_bits(p.scale, want_scale)) { std::puts("FAIL quantizer scale"); return 1; }
    // the packed codes must be what sym_quant gives for that scale
    auto q2 = duq::sym_quant(x.view({-1, K}), p.scale.view(-1));
    if (!torch::equal(q2, p.quantized_x.view({-1, K / 2}))) { std::puts("FAIL quantizer codes"); return 1; }

    // dual quantizer op: with equal scales it is the plain one; with different scales columns >= 10 follow scale_2
    auto sx1 = p.scale.view(-1);
    if (!torch::equal(duq::sym_dual_quant(x.view({-1, K}), sx1, sx1), q2)) { std::puts("FAIL sym_dual_quant equal scales"); return 1; }
    auto qd = duq::sym_dual_quant(x.view({-1, K}), sx1, sx1 * 2);
    auto qhalf = duq::sym_quant(x.view({-1, K}), sx1 * 2);
    if (!torch::equal(qd.slice(1, 0, 5), q2.slice(1, 0, 5)) || !torch::equal(qd.slice(1, 5), qhalf.slice(1, 5))) {
        std::puts("FAIL sym_dual_quant split"); return 1;
    }
    duq::PackedDoubleQuantizedTensor pd(qd, p.scale, p.scale * 2);
    if (pd.sizes() != qd.sizes()) { std::puts("FAIL PackedDoubleQuantizedTensor"); return 1; }

    auto l = duq::Linear4bit::from_float(lin, ws);
    auto y = l.forward(p);
    auto acc = duq::matmul(p.quantized_x.view({-1, K / 2}), l.weight);
    auto y3 = (duq::sym_dequant(acc, p.scale.view(-1), l.weight_scale.view(-1), 32) + l.bias).view({3, M / 3, N});
    if (!same_bits(y, y3)) { std::puts("FAIL Linear4bit fused vs three-step"); return 1; }

    // close to the fp16 layer it replaces (4-bit error, loose bound) - guards against a transposed operand
    auto yref = lin->forward(x).to(torch::kFloat32);
    auto rel = ((y.to(torch::kFloat32) - yref).norm() / yref.norm()).item<float>();
    if (!(rel < 0.35f)) { std::printf("FAIL Linear4bit vs fp16 layer: rel %.3f\n", rel); return 1; }

    auto ws1 = (w.slice(1, 0, 10).abs().amax(1, true).to(torch::kFloat32) / 7.0).to(torch::kHalf);
    auto d = duq::Linear4bitDUQ::from_float(lin, ws1, ws);
    auto yd = d.forward(p);
    auto yd3 = (duq::sym_dual_dequant(acc.copy_(duq::matmul(p.quantized_x.view({-1, K / 2}), d.weight)), p.scale.view(-1),
                                      d.weight_scale_1.view(-1), d.weight_scale_2.view(-1), 32) +
                d.bias).view({3, M / 3, N});
    if (!same_bits(yd, yd3)) { std::puts("FAIL Linear4bitDUQ fused vs three-step"); return 1; }

    // 6-bit float matrix path: large enough input (>= 32 tiles of 64 x 256), shadows on both sides, same bits
    if (K % 128 == 0 && N % 16 == 0) {
        const int64_t M2 = 64 * 32 * 256 / ((N + 255) / 256 * 256) + 64;
        auto x2 = (torch::randn({M2, K}, torch::dtype(torch::kFloat32).device(dev)) * 1.5).to(torch::kHalf);
        duq::Quantizer4bit quant6(1.0f, DUQ_QMAX_SYM_DEVICE, true);
        auto p6 = quant6.forward(x2);
        auto p4 = quant.forward(x2);
        if (!p6.shadow_x.defined() || p6.shadow_x.size(-1) != K * 3 / 4 || !torch::equal(p6.quantized_x, p4.quantized_x)) {
            std::puts("FAIL shadow quantizer"); return 1;
        }
        auto y4 = l.forward(p4);
        auto yd4 = d.forward(p4);
        l.enable_fp6();
        d.enable_fp6();
        if (!duq::detail::use_shadow(p6, l.weight_shadow, N)) { std::puts("FAIL 6-bit float path not taken"); return 1; }
        if (!same_bits(l.forward(p6), y4)) { std::puts("FAIL Linear4bit 6-bit float path vs integer path"); return 1; }
        if (!same_bits(d.forward(p6), yd4)) { std::puts("FAIL Linear4bitDUQ 6-bit float path vs integer path"); return 1; }
        if (!same_bits(l.forward(p4), y4)) { std::puts("FAIL Linear4bit without an activation shadow"); return 1; }
    }

    // decode: up to 64 rows are handed from Quantizer4bit to the layer unquantized and run in one library call (ONE
    // launch up to eight rows) (torch::nn::Sequential(Quantizer4bit, Linear4bit), test/pipeline.cu:107-110 of the
    // reference); same bits as the quantizer call followed by the GEMM call, and as the three steps
    if (K % 64 == 0) {
        duq::Quantizer4bit &eager = quant;
        duq::Quantizer4bit handover(1.0f, DUQ_QMAX_SYM_DEVICE, false, 64);
        for (int64_t rows : {1, 4, 8, 16, 64}) {
            if (rows > M) continue;
            auto xd = x.view({-1, K}).slice(0, 0, rows).contiguous().view({1, rows, K});
            auto pd8 = handover.forward(xd);
            if (!pd8.is_deferred() || pd8.sizes() != torch::IntArrayRef({1, rows, K / 2})) { std::puts("FAIL decode input not deferred"); return 1; }
            auto pe = eager.forward(xd);
            if (pe.is_deferred()) { std::puts("FAIL deferred by default"); return 1; }
            auto y1 = l.forward(pd8), y2 = l.forward(pe);
            auto acc8 = duq::matmul(pe.quantized_x.view({-1, K / 2}), l.weight);
            auto y38 = (duq::sym_dequant(acc8, pe.scale.view(-1), l.weight_scale.view(-1), 32) + l.bias).view({1, rows, N});
            if (!same_bits(y1, y2) || !same_bits(y1, y38)) { std::printf("FAIL Linear4bit decode, %ld rows\n", (long)rows); return 1; }
            if (!same_bits(d.forward(pd8), d.forward(pe))) { std::printf("FAIL Linear4bitDUQ decode, %ld rows\n", (long)rows); return 1; }
            pd8.materialize();
            if (pd8.is_deferred() || !torch::equal(pd8.quantized_x, pe.quantized_x) || !same_bits(pd8.scale, pe.scale)) {
                std::puts("FAIL materialize"); return 1;
            }
        }
        torch::nn::Sequential seq(duq::Quantizer4bit(1.0f, DUQ_QMAX_SYM_DEVICE, false, 64), duq::Linear4bit::from_float(lin, ws));
        auto xs = x.view({-1, K}).slice(0, 0, 3).contiguous();
        if (!same_bits(seq->forward(xs), l.forward(eager.forward(xs)))) { std::puts("FAIL Sequential decode"); return 1; }
    }

    bool threw = false;
    try { duq::sym_dequant(acc, p.scale.view(-1), l.weight_scale.view(-1), 16); } catch (const c10::Error &) { threw = true; }
    if (!threw) { std::puts("FAIL bits != 32 accepted"); return 1; }
    threw = false;
    try { quant.forward(x.to(torch::kBFloat16)); } catch (const c10::Error &) { threw = true; }
    if (!threw) { std::puts("FAIL bf16 accepted"); return 1; }

    torch::cuda::synchronize();
    std::printf("OK %.6f rel %.4f\n", y.to(torch::kFloat32).abs().sum().item<float>(), rel);
    return 0;
}

// C++ harness: replays forward_qmm / backward_qmm (include/llmq_qmm.hpp) for one linear layer on the
// GPU through the C++ shim (plus the SwiGLU activation on the projection output) and compares every result with the CPU oracle (oracle/llmq_oracle.c, linked
// into this test binary only).  Also exercises the shim's exception behaviour.
//   usage: qmm_harness BT C OC [reuse_inp]
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "llmq_qmm.hpp"

extern "C" {
float orc_abs_max_bf16(const uint16_t* in, int64_t n);
float orc_bf16_to_f32(uint16_t h);
void orc_quantize_e4m3_bf16(uint8_t* out, float* scale_out, const uint16_t* in, float absmax, int64_t n);
void orc_transpose_u8(uint8_t* dst, const uint8_t* src, int rows, int cols);
void orc_gemm_tn_e4m3_exact_sampled(double* exact, double* sumabs, const uint8_t* a, const uint8_t* b, int M, int N, int K,
                                    const int32_t* idx_n, const int32_t* idx_m, int64_t count);
void orc_fill_normal_bf16(uint16_t* out, int64_t n, uint64_t seed, uint64_t stream, float mean, float std);
void orc_swiglu_forward_bf16(uint16_t* out, double* exact_out, const uint16_t* inp, int64_t BT, int C);
void orc_swiglu_forward_f32(float* out, double* exact_out, const float* inp, int64_t BT, int C);
float orc_abs_max_f32(const float* in, int64_t n);
void orc_backward_bias_bf16(uint16_t* dbias, const void* dout, int fmt, const float* sa, const float* sb, int64_t BT, int OC, double* colsum, double* colabs);
}

#define HIP_OK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { std::printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); return 2; } } while (0)

static int failures = 0;
#define EXPECT(cond, ...) do { if (!(cond)) { ++failures; std::printf("FAIL: " __VA_ARGS__); std::printf("\n"); } } while (0)

template <class T> static T* dalloc(std::size_t n) { void* p = nullptr; if (hipMalloc(&p, n * sizeof(T) + 16) != hipSuccess) std::abort(); return (T*)p; }

static Tensor make(ETensorDType dt, void* p, std::vector<long> shape, float* stats = nullptr) {
    Tensor t = Tensor::from_pointer((std::byte*)p, 0, dt, shape);
    t.Stats = stats;
    return t;
}

// old: values c held before an accumulating matmul (empty: none), decoded to double
static void check_gemm(const char* name, const std::vector<uint16_t>& got_bf16, const std::vector<float>& got_f32, int N, int M,
                       const uint8_t* a, const uint8_t* b, int K, float scale, const std::vector<double>& old = {}) {
    const int S = 20000;
    std::vector<int32_t> in(S), im(S);
    uint64_t s = 88172645463325252ull;
    for (int i = 0; i < S; ++i) { s ^= s << 13; s ^= s >> 7; s ^= s << 17; in[i] = (int32_t)(s % N); im[i] = (int32_t)((s >> 32) % M); }
    std::vector<double> ex(S), sa(S);
    orc_gemm_tn_e4m3_exact_sampled(ex.data(), sa.data(), a, b, M, N, K, in.data(), im.data(), S);
    double worst = 0, e2 = 0, r2 = 0, maxabs = 0;
    const bool bf16 = !got_bf16.empty();
    for (int i = 0; i < S; ++i) {
        const std::size_t o = (std::size_t)in[i] * M + im[i];
        const double g = bf16 ? (double)orc_bf16_to_f32(got_bf16[o]) : (double)got_f32[o];
        const double ref = ex[i] * scale + (old.empty() ? 0.0 : old[o]), err = std::fabs(g - ref);
        const double bound = std::ldexp(std::fabs(ref), bf16 ? -8 : -23) + std::ldexp(scale * sa[i], -11) + 1e-38;
        worst = std::fmax(worst, err / bound); maxabs = std::fmax(maxabs, err); e2 += err * err; r2 += ref * ref;
    }
    const double fro = std::sqrt(e2 / r2);
    std::printf("%-10s [%d x %d] K=%d: max-abs err %.3e, rel-Frobenius %.3e, worst/bound %.3f\n", name, N, M, K, maxabs, fro, worst);
    EXPECT(worst <= 1.0, "%s exceeds the element bound", name);
    EXPECT(fro <= (bf16 ? 2.5e-3 : 2e-4), "%s exceeds the Frobenius bound", name);
}

int main(int argc, char** argv) {
    const int BT = argc > 1 ? std::atoi(argv[1]) : 1024, C = argc > 2 ? std::atoi(argv[2]) : 896, OC = argc > 3 ? std::atoi(argv[3]) : 1152;
    const bool reuse_inp = argc > 4 && std::atoi(argv[4]) != 0;
    const bool fuse = argc > 5 && std::atoi(argv[5]) != 0;   // gradient quantize + transpose from one read
    // 1: bf16 weight gradient; 2: also ask for operands in their stored layouts (matmul modes NN / TT / NT) where the
    // plan expects them to pay; 3: wherever the shapes are served; 4 / 5: as 2 / 3 with an fp32 weight gradient
    const int dw_mode = argc > 6 ? std::atoi(argv[6]) : 0;
    const bool dw_bf16 = dw_mode >= 1 && dw_mode <= 3, direct = dw_mode >= 2, wherever = dw_mode == 3 || dw_mode == 5;
    // gradient accumulation: dweight starts from given values and the weight-gradient matmul adds to them
    const bool accumulate = argc > 7 && std::atoi(argv[7]) != 0;
    const int B = 1, T = BT;
    std::printf("qmm_harness BT=%d C=%d OC=%d reuse_inp=%d fuse=%d dweight=%s direct_grad_layout=%d wherever_served=%d accumulate=%d\n", BT, C, OC,
                (int)reuse_inp, (int)fuse, dw_bf16 ? "bf16" : "fp32", (int)direct, (int)wherever, (int)accumulate);
    hipStream_t stream; HIP_OK(hipStreamCreate(&stream));
    QmmRunState rs; HIP_OK(hipGetDeviceProperties(&rs.DeviceProp, 0));
    rs.FuseGradTranspose = fuse;
    rs.DirectGradLayout = direct;
    rs.DirectGradLayoutWhereverServed = wherever;
    const QmmRunState::DirectPlan plan =
        direct ? QmmRunState::direct_layout_plan(B, T, C, OC, ETensorDType::BF16, dw_bf16 ? ETensorDType::BF16 : ETensorDType::FP32, accumulate,
                                                 wherever)
               : QmmRunState::DirectPlan{};
    std::printf("stored-layout plan: dgrad in place %d, wgrad %s\n", (int)plan.DgradInPlace,
                plan.Wgrad == QmmRunState::EWgrad::Copies ? "copies" : plan.Wgrad == QmmRunState::EWgrad::GradInPlace ? "gradient in place (TT)"
                                                                                                                    : "both in place (NT)");
    rs.Capacity = QmmRunState::backward_temp_bytes(B, T, C, OC, fuse, plan);
    rs.Arena = dalloc<std::byte>(rs.Capacity);

    std::vector<uint16_t> hx((std::size_t)BT * C), hw((std::size_t)OC * C), hdy((std::size_t)BT * OC);
    orc_fill_normal_bf16(hx.data(), hx.size(), 7, 1, 0.f, 1.f);
    orc_fill_normal_bf16(hw.data(), hw.size(), 7, 2, 0.f, 0.02f);
    orc_fill_normal_bf16(hdy.data(), hdy.size(), 7, 3, 0.f, 1e-3f);
    auto* dx = dalloc<uint16_t>(hx.size()); auto* dw = dalloc<uint16_t>(hw.size()); auto* ddy = dalloc<uint16_t>(hdy.size());
    HIP_OK(hipMemcpy(dx, hx.data(), hx.size() * 2, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(dw, hw.data(), hw.size() * 2, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(ddy, hdy.data(), hdy.size() * 2, hipMemcpyHostToDevice));
    float* stats = dalloc<float>(8);   // [x: absmax, scale][w][dy]
    HIP_OK(hipMemset(stats, 0, 32));

    QuantizableTensor inp{make(ETensorDType::BF16, dx, {BT, C}), make(ETensorDType::FP8_E4M3, dalloc<uint8_t>(hx.size()), {BT, C}, stats)};
    QuantizableTensor dout{make(ETensorDType::BF16, ddy, {BT, OC}), make(ETensorDType::FP8_E4M3, dalloc<uint8_t>(hdy.size()), {BT, OC}, stats + 4)};
    Tensor w_master = make(ETensorDType::BF16, dw, {OC, C});
    Tensor weight = make(ETensorDType::FP8_E4M3, dalloc<uint8_t>(hw.size()), {OC, C}, stats + 2);
    Tensor out = make(ETensorDType::BF16, dalloc<uint16_t>((std::size_t)BT * OC), {BT, OC});
    Tensor dinp = make(ETensorDType::BF16, dalloc<uint16_t>((std::size_t)BT * C), {BT, C});
    Tensor dweight = dw_bf16 ? make(ETensorDType::BF16, dalloc<uint16_t>((std::size_t)OC * C), {OC, C})
                             : make(ETensorDType::FP32, dalloc<float>((std::size_t)OC * C), {OC, C});
    Tensor no_bias{};
    // matmul workspace sized like the reference's (src/training/model.cpp:69)
    Tensor workspace = make(ETensorDType::BYTE, dalloc<uint8_t>(32u << 20), {32L << 20});
    rs.Workspace = workspace;

    // producers' abs-max epilogues are replaced by the standalone kernel; weights as llama_weights.cpp:207-223
    abs_max(inp.Quant.abs_max(), inp.Value, (long)BT * C, rs.DeviceProp, stream);
    abs_max(weight.abs_max(), w_master, (long)OC * C, rs.DeviceProp, stream);
    abs_max(dout.Quant.abs_max(), dout.Value, (long)BT * OC, rs.DeviceProp, stream);
    quantize_with_abs_max(weight, weight.scale(), w_master, weight.abs_max(), (long)OC * C, rs.DeviceProp, stream);
    forward_qmm(out, inp, weight, no_bias, nullptr, workspace, B, T, C, OC, rs.DeviceProp, false, stream, EMatmulBackend::Custom);
    // bias gradient of the layer (the QKV projection has one): starts from a non-zero value, as an accumulated gradient
    std::vector<uint16_t> hdb0(OC);
    orc_fill_normal_bf16(hdb0.data(), hdb0.size(), 7, 4, 0.f, 1e-2f);
    Tensor dbias = make(ETensorDType::BF16, dalloc<uint16_t>(OC), {OC});
    HIP_OK(hipMemcpy(dbias.Data, hdb0.data(), (std::size_t)OC * 2, hipMemcpyHostToDevice));
    const int bias_scratch = get_bias_backward_scratch_size(ETensorDType::FP8_E4M3, OC, rs.DeviceProp);   // dtype of the gradient it sums
    Tensor bias_buffer = make(ETensorDType::FP32, dalloc<float>((std::size_t)bias_scratch / 4), {bias_scratch / 4});
    // the weight gradient an accumulating micro-step starts from
    std::vector<double> dw_old;
    if (accumulate) {
        std::vector<uint16_t> h0((std::size_t)OC * C);
        orc_fill_normal_bf16(h0.data(), h0.size(), 7, 5, 0.f, 1e-3f);
        dw_old.resize(h0.size());
        for (std::size_t i = 0; i < h0.size(); ++i) dw_old[i] = (double)orc_bf16_to_f32(h0[i]);
        if (dw_bf16) {
            HIP_OK(hipMemcpy(dweight.Data, h0.data(), h0.size() * 2, hipMemcpyHostToDevice));
        } else {
            std::vector<float> f0(h0.size());
            for (std::size_t i = 0; i < h0.size(); ++i) f0[i] = orc_bf16_to_f32(h0[i]);
            HIP_OK(hipMemcpy(dweight.Data, f0.data(), f0.size() * 4, hipMemcpyHostToDevice));
        }
    }
    backward_qmm(dinp, dweight, dbias, dout, inp, weight, bias_buffer, accumulate, rs, B, T, C, OC, reuse_inp, stream);
    HIP_OK(hipStreamSynchronize(stream));
    EXPECT(rs.Top == 0 && rs.Live.empty(), "temporary stack not unwound");
    EXPECT(rs.HighWater == rs.Capacity, "backward_temp_bytes (%zu) != high-water mark (%zu)", rs.Capacity, rs.HighWater);

    // ---- oracle side ----
    float hstats[8]; HIP_OK(hipMemcpy(hstats, stats, 32, hipMemcpyDeviceToHost));
    const float ax = orc_abs_max_bf16(hx.data(), hx.size()), aw = orc_abs_max_bf16(hw.data(), hw.size()), ag = orc_abs_max_bf16(hdy.data(), hdy.size());
    std::vector<uint8_t> xq(hx.size()), wq(hw.size()), gq(hdy.size());
    float sx, sw, sg;
    orc_quantize_e4m3_bf16(xq.data(), &sx, hx.data(), ax, hx.size());
    orc_quantize_e4m3_bf16(wq.data(), &sw, hw.data(), aw, hw.size());
    orc_quantize_e4m3_bf16(gq.data(), &sg, hdy.data(), ag, hdy.size());
    EXPECT(std::memcmp(&hstats[0], &ax, 4) == 0 && std::memcmp(&hstats[2], &aw, 4) == 0 && std::memcmp(&hstats[4], &ag, 4) == 0, "abs-max mismatch");
    EXPECT(std::memcmp(&hstats[1], &sx, 4) == 0 && std::memcmp(&hstats[3], &sw, 4) == 0 && std::memcmp(&hstats[5], &sg, 4) == 0, "scale mismatch");
    std::vector<uint8_t> got(std::max({xq.size(), wq.size(), gq.size()}));
    HIP_OK(hipMemcpy(got.data(), inp.Quant.Data, xq.size(), hipMemcpyDeviceToHost));
    EXPECT(std::memcmp(got.data(), xq.data(), xq.size()) == 0, "x quantized bytes differ");
    HIP_OK(hipMemcpy(got.data(), weight.Data, wq.size(), hipMemcpyDeviceToHost));
    EXPECT(std::memcmp(got.data(), wq.data(), wq.size()) == 0, "w quantized bytes differ");
    HIP_OK(hipMemcpy(got.data(), dout.Quant.Data, gq.size(), hipMemcpyDeviceToHost));
    EXPECT(std::memcmp(got.data(), gq.data(), gq.size()) == 0, "dy quantized bytes differ");

    std::vector<uint16_t> hy((std::size_t)BT * OC), hdx((std::size_t)BT * C), hdw16; std::vector<float> hdw;
    if (dw_bf16) hdw16.resize((std::size_t)OC * C); else hdw.resize((std::size_t)OC * C);
    HIP_OK(hipMemcpy(hy.data(), out.Data, hy.size() * 2, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(hdx.data(), dinp.Data, hdx.size() * 2, hipMemcpyDeviceToHost));
    if (dw_bf16) HIP_OK(hipMemcpy(hdw16.data(), dweight.Data, hdw16.size() * 2, hipMemcpyDeviceToHost));
    else HIP_OK(hipMemcpy(hdw.data(), dweight.Data, hdw.size() * 4, hipMemcpyDeviceToHost));
    std::vector<uint8_t> wqt(wq.size()), xqt(xq.size()), gqt(gq.size());
    orc_transpose_u8(wqt.data(), wq.data(), OC, C);
    orc_transpose_u8(xqt.data(), xq.data(), BT, C);
    orc_transpose_u8(gqt.data(), gq.data(), BT, OC);
    check_gemm("forward", hy, {}, BT, OC, wq.data(), xq.data(), C, sw * sx);
    check_gemm("dgrad", hdx, {}, BT, C, wqt.data(), gq.data(), OC, sw * sg);
    check_gemm("wgrad", hdw16, hdw, OC, C, xqt.data(), gqt.data(), BT, sx * sg, dw_old);

    {   // dbias += sx*sg * column sums of the quantized gradient (llama_model.cpp:334-336)
        std::vector<uint16_t> hdb(OC), want(hdb0);
        std::vector<double> cs(OC), ca(OC);
        HIP_OK(hipMemcpy(hdb.data(), dbias.Data, (std::size_t)OC * 2, hipMemcpyDeviceToHost));
        orc_backward_bias_bf16(want.data(), gq.data(), 0, &sx, &sg, BT, OC, cs.data(), ca.data());
        double worst = 0;
        for (int oc = 0; oc < OC; ++oc) {
            const double ref = cs[oc] * (double)(sx * sg) + (double)orc_bf16_to_f32(hdb0[oc]);
            const double bound = std::ldexp(std::fabs(ref), -8) + std::ldexp((double)(sx * sg) * ca[oc], -18) + 1e-30;
            worst = std::max(worst, std::fabs((double)orc_bf16_to_f32(hdb[oc]) - ref) / bound);
        }
        std::printf("%-8s worst error / bound %.3f\n", "dbias", worst);
        EXPECT(worst <= 1.0, "dbias exceeds the element bound");
    }

    if (OC % 16 == 0) {
        // The projection's output as the [up | gate] input of the activation in front of the next matmul
        // (llama_model.cpp:216 and :613-617): swiglu_forward with its abs-max, then the e4m3 codes either by
        // quantize_with_abs_max or directly by swiglu_forward_quant -- the same bytes.
        const int D = OC / 2;
        const std::size_t n = (std::size_t)BT * D;
        float* hstat = dalloc<float>(4);
        Tensor act = make(ETensorDType::BF16, dalloc<uint16_t>(n), {BT, D});
        Tensor act_q = make(ETensorDType::FP8_E4M3, dalloc<uint8_t>(n), {BT, D}, hstat);
        Tensor act_q2 = make(ETensorDType::FP8_E4M3, dalloc<uint8_t>(n), {BT, D}, hstat + 2);
        swiglu_forward(act, out, act_q.abs_max(), B, T, D, stream);
        quantize_with_abs_max(act_q, act_q.scale(), act, act_q.abs_max(), (long)n, rs.DeviceProp, stream);
        swiglu_forward_quant(act_q2, act_q2.scale(), out, act_q.abs_max(), B, T, D, stream);
        HIP_OK(hipStreamSynchronize(stream));
        std::vector<uint16_t> hact(n), want(n);
        std::vector<double> exact(n);
        std::vector<uint8_t> q1(n), q2(n), qo(n);
        float st[4];
        HIP_OK(hipMemcpy(hact.data(), act.Data, n * 2, hipMemcpyDeviceToHost));
        HIP_OK(hipMemcpy(q1.data(), act_q.Data, n, hipMemcpyDeviceToHost));
        HIP_OK(hipMemcpy(q2.data(), act_q2.Data, n, hipMemcpyDeviceToHost));
        HIP_OK(hipMemcpy(st, hstat, 16, hipMemcpyDeviceToHost));
        orc_swiglu_forward_bf16(want.data(), exact.data(), hy.data(), BT, D);
        double worst = 0;
        for (std::size_t i = 0; i < n; ++i)
            worst = std::fmax(worst, std::fabs((double)orc_bf16_to_f32(hact[i]) - (double)orc_bf16_to_f32(want[i])) /
                                         (std::ldexp(std::fabs(exact[i]), -7) + 1e-38));
        std::printf("%-10s [%d x %d]: worst error / (one bf16 ulp) %.3f\n", "swiglu", BT, D, worst);
        EXPECT(worst <= 1.0, "swiglu_forward is more than one bf16 ulp from the oracle");
        const float aa = orc_abs_max_bf16(hact.data(), n);
        float sq;
        orc_quantize_e4m3_bf16(qo.data(), &sq, hact.data(), aa, n);
        EXPECT(std::memcmp(&st[0], &aa, 4) == 0, "swiglu abs-max differs from the abs-max of its output");
        EXPECT(std::memcmp(&st[1], &sq, 4) == 0 && std::memcmp(&st[3], &sq, 4) == 0, "swiglu quantization scales differ");
        EXPECT(std::memcmp(q1.data(), qo.data(), n) == 0, "quantized activation differs from the oracle");
        EXPECT(std::memcmp(q1.data(), q2.data(), n) == 0, "swiglu_forward_quant differs from swiglu_forward + quantize");
        {   // the fp32 overload through the same Tensor entry (an fp32 model in front of FP8 matmuls): the same input as fp32
            std::vector<float> hin((std::size_t)BT * OC), hout(n);
            for (std::size_t i = 0; i < hin.size(); ++i) hin[i] = orc_bf16_to_f32(hy[i]) * 1.0009765625f;
            Tensor in32 = make(ETensorDType::FP32, dalloc<float>(hin.size()), {BT, OC});
            Tensor out32 = make(ETensorDType::FP32, dalloc<float>(n), {BT, D});
            HIP_OK(hipMemcpy(in32.Data, hin.data(), hin.size() * 4, hipMemcpyHostToDevice));
            swiglu_forward(out32, in32, hstat, B, T, D, stream);
            HIP_OK(hipStreamSynchronize(stream));
            float am32;
            HIP_OK(hipMemcpy(hout.data(), out32.Data, n * 4, hipMemcpyDeviceToHost));
            HIP_OK(hipMemcpy(&am32, hstat, 4, hipMemcpyDeviceToHost));
            std::vector<float> want32(n);
            orc_swiglu_forward_f32(want32.data(), exact.data(), hin.data(), BT, D);
            double worst32 = 0;
            for (std::size_t i = 0; i < n; ++i)
                worst32 = std::fmax(worst32, std::fabs((double)hout[i] - exact[i]) / (std::ldexp(std::fabs(exact[i]), -23) + 1e-37));
            std::printf("%-10s [%d x %d]: worst error / (one fp32 ulp) %.3f\n", "swiglu f32", BT, D, worst32);
            EXPECT(worst32 <= 4.0, "fp32 swiglu_forward is more than four fp32 ulp from the oracle");
            const float aa32 = orc_abs_max_f32(hout.data(), n);
            EXPECT(std::memcmp(&am32, &aa32, 4) == 0, "fp32 swiglu abs-max differs from the abs-max of its output");
        }
        bool sw_threw = false;
        try { swiglu_forward(act, out, nullptr, B, T, D + 4, stream); }
        catch (const std::invalid_argument&) { sw_threw = true; }
        EXPECT(sw_threw, "swiglu_forward with C %% 8 != 0 must throw std::invalid_argument");
    }

    {   // weight side: e4m3 copies rebuilt only when the layer or the optimizer version changes (llama_weights.cpp:434-504)
        float* wstats = dalloc<float>(2);
        Tensor master = make(ETensorDType::BF16, dw, {OC, C}, wstats);
        abs_max(master.abs_max(), master, (long)OC * C, rs.DeviceProp, stream);
        QuantizedWeightCache cache({make(ETensorDType::FP8_E4M3, dalloc<uint8_t>(hw.size()), {OC, C}),
                                    make(ETensorDType::FP8_E4M3, dalloc<uint8_t>(hw.size()), {OC, C})});
        cache.get(0, master, rs.DeviceProp, stream);
        cache.get(1, master, rs.DeviceProp, stream);
        Tensor& again = cache.get(0, master, rs.DeviceProp, stream);
        EXPECT(cache.quantize_calls() == 2, "cached layer was requantized");
        cache.get(2, master, rs.DeviceProp, stream);          // takes layer 0's slot
        cache.get(0, master, rs.DeviceProp, stream);
        EXPECT(cache.quantize_calls() == 4, "evicted layer was not requantized");
        cache.invalidate();                                   // optimizer step
        Tensor& fresh = cache.get(1, master, rs.DeviceProp, stream);
        EXPECT(cache.quantize_calls() == 5, "stale version was not requantized");
        HIP_OK(hipStreamSynchronize(stream));
        float ws2[2]; HIP_OK(hipMemcpy(ws2, wstats, 8, hipMemcpyDeviceToHost));
        EXPECT(std::memcmp(&ws2[0], &aw, 4) == 0 && std::memcmp(&ws2[1], &sw, 4) == 0, "weight cache: abs-max / scale mismatch");
        EXPECT(fresh.scale() == master.scale() && again.abs_max() == master.abs_max(), "weight cache: Stats not shared with the master");
        HIP_OK(hipMemcpy(got.data(), fresh.Data, wq.size(), hipMemcpyDeviceToHost));
        EXPECT(std::memcmp(got.data(), wq.data(), wq.size()) == 0, "weight cache: quantized bytes differ");
    }

    // ---- error behaviour of the shim (reference: matmul.cpp:55-57, kernels.cpp:18-24) ----
    bool threw = false;
    try { matmul(out, weight, inp.Quant, no_bias, nullptr, nullptr, nullptr, workspace, OC, BT, C + 8, EMMTranspose::TN, false, stream); }
    catch (const std::invalid_argument&) { threw = true; }
    EXPECT(threw, "matmul with K %% 16 != 0 (operand rows not 16-byte aligned) must throw std::invalid_argument");
    threw = false;
    try { matmul(out, weight, inp.Quant, no_bias, nullptr, nullptr, nullptr, workspace, OC, BT, C + 16, EMMTranspose::NN, false, stream); }
    catch (const std::invalid_argument&) { threw = true; }
    EXPECT(threw, "FP8 matmul in mode NN off the 256 lattice (not served) must throw std::invalid_argument");
    threw = false;
    try { quantize_with_abs_max(out, nullptr, inp.Value, stats, 8, rs.DeviceProp, stream); }
    catch (const std::invalid_argument&) { threw = true; }
    EXPECT(threw, "unsupported dtype combination must throw std::invalid_argument");

    std::printf(failures ? "RESULT: FAIL (%d)\n" : "RESULT: PASS\n", failures);
    return failures ? 1 : 0;
}

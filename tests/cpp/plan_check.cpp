// Host-only check of QmmRunState::direct_layout_plan and backward_temp_bytes (no GPU, no library call): which
// backward matmuls of a layer read their operands in the stored layout, and what stack that leaves.
#include <cstdio>
#include <cstdlib>

#include "llmq_qmm.hpp"

static int failures = 0;
#define EXPECT(cond, ...) do { if (!(cond)) { ++failures; std::printf("FAIL: " __VA_ARGS__); std::printf("\n"); } } while (0)

static void expect_plan(const char* what, int BT, int C, int OC, ETensorDType dinp, ETensorDType dw, bool accumulate, bool wherever,
                        bool dgrad, EQmmWgrad wgrad) {
    const QmmDirectPlan p = QmmRunState::direct_layout_plan(1, BT, C, OC, dinp, dw, accumulate, wherever);
    EXPECT(p.DgradInPlace == dgrad && p.Wgrad == wgrad, "%s: BT=%d C=%d OC=%d -> dgrad %d wgrad %d", what, BT, C, OC,
           (int)p.DgradInPlace, (int)p.Wgrad);
}

int main() {
    const ETensorDType BF = ETensorDType::BF16, F32 = ETensorDType::FP32;
    using W = EQmmWgrad;
    // Qwen2.5-7B MLP at 8192 tokens: down projection (C = 18944 -> OC = 3584) NN + NT, gate+up (3584 -> 37888) NN + TT
    expect_plan("7B down", 8192, 18944, 3584, BF, BF, false, false, true, W::BothInPlace);
    expect_plan("7B gate+up", 8192, 3584, 37888, BF, BF, false, false, true, W::GradInPlace);
    // at 4096 tokens the dgrad keeps its copy; the weight gradients still read in place
    expect_plan("7B down, 4096 tokens", 4096, 18944, 3584, BF, BF, false, false, false, W::BothInPlace);
    expect_plan("7B gate+up, 4096 tokens", 4096, 3584, 37888, BF, BF, false, false, false, W::GradInPlace);
    // Qwen2.5-1.5B (1536 / 8960): small weights -> copying dgrad
    expect_plan("1.5B down", 16384, 8960, 1536, BF, BF, false, false, false, W::BothInPlace);
    expect_plan("1.5B gate+up", 16384, 1536, 17920, BF, BF, false, false, false, W::GradInPlace);
    // accumulation (gradient-accumulation micro-steps) and fp32 weight gradients are served in place as well
    expect_plan("accumulate, small C", 8192, 3584, 37888, BF, BF, true, false, true, W::GradInPlace);
    expect_plan("accumulate, large C and large weight", 8192, 18944, 3584, BF, BF, true, false, true, W::Copies);
    expect_plan("accumulate, large weight, wherever served", 8192, 18944, 3584, BF, BF, true, true, true, W::BothInPlace);
    expect_plan("fp32 dweight", 8192, 18944, 3584, BF, F32, false, false, true, W::BothInPlace);
    expect_plan("fp32 dweight, accumulate", 8192, 18944, 3584, BF, F32, true, false, true, W::Copies);
    expect_plan("fp32 dweight, gate+up", 8192, 3584, 37888, BF, F32, true, false, true, W::GradInPlace);
    expect_plan("1.5B down, fp32 dweight, accumulate", 16384, 8960, 1536, BF, F32, true, false, false, W::BothInPlace);
    // an fp32 dinp is not served in place
    expect_plan("fp32 dinp", 8192, 18944, 3584, F32, BF, false, false, false, W::BothInPlace);
    // Qwen2.5-0.5B (C = 896 = 4 x 224): only the gradient in place, on 224-wide tiles (bf16 output without accumulation)
    expect_plan("0.5B gate+up", 8192, 896, 9728, BF, BF, false, false, false, W::GradInPlace);
    expect_plan("0.5B gate+up, accumulate", 8192, 896, 9728, BF, BF, true, false, false, W::Copies);
    expect_plan("0.5B gate+up, fp32 dweight", 8192, 896, 9728, BF, F32, false, false, false, W::Copies);
    // 0.5B down (C = 4864 = 19 x 256, OC = 896): OC off the 256 lattice -> copies
    expect_plan("0.5B down, fp32 dweight", 8192, 4864, 896, BF, F32, false, false, false, W::Copies);
    // off the 256 lattice: nothing
    expect_plan("OC = 1152", 1024, 896, 1152, BF, BF, false, false, false, W::Copies);
    expect_plan("BT = 1000", 1000, 1024, 1024, BF, BF, false, true, false, W::Copies);
    // wherever served: thresholds ignored, limits kept
    expect_plan("small layer, wherever served", 1024, 1024, 1536, BF, BF, false, true, true, W::BothInPlace);
    expect_plan("large OC, wherever served", 1024, 768, 9216, BF, BF, false, true, true, W::BothInPlace);
    expect_plan("operand of 2 GiB", 65536, 32768, 1024, BF, BF, false, true, true, W::GradInPlace);   // BT * C = 2^31: not NT
    expect_plan("gradient of 2 GiB", 65536, 1024, 32768, BF, BF, false, true, true, W::Copies);        // BT * OC = 2^31

    // stack of one layer, bytes (every block rounded up to 4096): reference sequence max(C * OC, BT * (C + OC));
    // in place nothing of what the plan drops
    const long BT = 8192, C = 18944, OC = 3584;
    const std::size_t ref = QmmRunState::backward_temp_bytes(1, BT, C, OC);
    EXPECT(ref == (std::size_t)(BT * C + BT * OC), "reference stack %zu", ref);
    const QmmDirectPlan nn_nt = QmmRunState::direct_layout_plan(1, BT, C, OC, BF, BF, false);
    EXPECT(QmmRunState::backward_temp_bytes(1, BT, C, OC, false, nn_nt) == 0, "NN + NT keeps %zu bytes",
           QmmRunState::backward_temp_bytes(1, BT, C, OC, false, nn_nt));
    QmmDirectPlan tt;
    tt.Wgrad = W::GradInPlace;
    EXPECT(QmmRunState::backward_temp_bytes(1, BT, C, OC, false, tt) == (std::size_t)(BT * C), "TT with copying dgrad");
    EXPECT(QmmRunState::backward_temp_bytes(1, BT, C, OC, true) == (std::size_t)(BT * OC + BT * C), "fused, reference sequence");
    std::printf(failures ? "RESULT: FAIL (%d)\n" : "RESULT: PASS\n", failures);
    return failures ? 1 : 0;
}

// llmq_qmm.hpp -- host glue that issues the kernel call sequence of one FP8 linear layer, forward and
// backward, the way the reference's forward_qmm / backward_qmm do (src/models/llama_model.cpp:25-47,
// 280-340, FP8 branches).  The reference passes its whole LLamaRunState into backward_qmm; here the
// part of it the path needs (a LIFO device stack for temporaries, the device properties and the
// gradient dtype, src/training/model.cpp:129-143, src/utilities/stack.cpp:13-25) is QmmRunState.
#ifndef LLMQ_QMM_HPP
#define LLMQ_QMM_HPP

#include "llmq_kernels.hpp"

// What backward_qmm does about the transposed copies of its matmul operands (QmmRunState::DirectGradLayout).
enum class EQmmWgrad { Copies, GradInPlace, BothInPlace };   // reference sequence; mode TT; mode NT
struct QmmDirectPlan {
    bool DgradInPlace = false;   // dgrad reads weight[OC, C] as the K-major first operand (mode NN): no weight_tp
    EQmmWgrad Wgrad = EQmmWgrad::Copies;
};

// LIFO bump allocator over one device arena: temp_alloc / temp_free are host pointer arithmetic only,
// so the sequence stays legal under stream capture.  Blocks are rounded up to 4096 bytes.
struct QmmRunState {
    std::byte* Arena = nullptr;
    std::size_t Capacity = 0;
    std::size_t Top = 0;
    std::size_t HighWater = 0;
    int Device = 0;
    hipDeviceProp_t DeviceProp{};
    ETensorDType GradDType = ETensorDType::FP8_E4M3;
    llmqBlasHandle_t BlasHandle = nullptr;
    Tensor Workspace{};
    EMatmulBackend MatmulBackend = EMatmulBackend::Custom;
    // Extension: quantize the output gradient and produce its transpose from one read of dout.Value (saves one
    // read and one launch per layer; the transposed gradient then lives on the stack during the dgrad as well).
    bool FuseGradTranspose = false;
    // Extension: backward_qmm hands the matmuls their operands where they lie (matmul modes NN / TT / NT) instead of
    // transposed copies, wherever direct_layout_plan() finds the shapes served and the copy dearer than the mode's
    // slower K loop; elsewhere it behaves as without the flag.
    bool DirectGradLayout = false;
    // With DirectGradLayout: take every stored-layout mode the shapes allow, whatever it costs in time (the transposed
    // copies then never occupy the stack: backward_temp_bytes() shrinks accordingly).
    bool DirectGradLayoutWhereverServed = false;
    using EWgrad = EQmmWgrad;
    using DirectPlan = QmmDirectPlan;
    // The K-major modes serve whole 256-wide tiles and operands below 2 GiB (bf16 and fp32 output, with accumulation;
    // a K-major first operand with fp32 output or accumulation takes a slower, fp32-staged epilogue).  Which of them pay
    // was measured on MLP layers of Qwen2.5-7B (C = 3584, FFN 18944), 1.5B (1536, 8960)
    // and a 2048 / 8192 layer at 4096 to 16384 tokens, every matmul with the 32 MiB workspace, against mode TN plus the
    // byte transposes it needs (2 bytes moved per element copied):
    //  * weight gradient: on the 7B layers a K-major second operand costs 3-4 % of the matmul and both operands K-major
    //    2-9 % (up to 20 % on the 1.5B layers, whose small outputs mode TN serves with plans of its own); the copies
    //    cost more on every layer measured (7B at 8192 tokens: 442 -> 389 us in mode NT, 862 -> 778 us in mode TT with
    //    the activation's copy; 1.5B at 16384 tokens: 207 -> 181 us and 422 -> 340 us).  NT where the activation is the
    //    larger copy (OC <= 8192), else TT while the matmul stays small enough (C <= 8192).
    //  * dgrad in mode NN saves only the weight's copy (26 and 45 us on the 7B layers, 7-11 us on the 1.5B ones) and has
    //    one tile plan (256 x 256, bf16 staged through LDS) where mode TN picks 224- or 192-wide tiles or a small-output
    //    plan: level with TN per tile on the 7B down projection from 8192 tokens on (439 -> 415 us, 760 -> 750 us for
    //    gate+up), 13-16 % slower at 4096 tokens, 20-48 % slower on the 1.5B and 2048-wide layers (short K, few tiles).
    //    Taken for weights of 48 M elements and more at 8192 to 16384 tokens.
    static DirectPlan direct_layout_plan(int B, int T, int C, int OC, ETensorDType dinp_dtype, ETensorDType dweight_dtype,
                                         bool accumulate, bool wherever_served = false) {
        const long BT = (long)B * T, lim = 1L << 31;
        const bool tiles = C % 256 == 0 && OC % 256 == 0 && BT % 256 == 0;
        DirectPlan p;
        p.DgradInPlace = tiles && dinp_dtype == ETensorDType::BF16 && (long)C * OC < lim &&
                         (wherever_served || ((long)C * OC >= (48L << 20) && BT >= 8192 && BT <= 16384));
        const bool bf16_dw = dweight_dtype == ETensorDType::BF16;
        if ((bf16_dw || dweight_dtype == ETensorDType::FP32) && OC % 256 == 0 && BT % 256 == 0 && BT * OC < lim) {
            // accumulating into c with both operands K-major costs the fp32-staged epilogue a read of the old values in
            // 8- or 16-byte pieces: measured ahead of the copies on the 1.5B layers (184 against 238 us, 436 against 485 us
            // into fp32), behind them on the 7B ones (533 against 512 us): taken for weights up to 32 M elements
            const bool nt_pays = !accumulate || (long)C * OC <= (32L << 20);
            if (tiles && BT * C < lim && (wherever_served || (OC <= 8192 && nt_pays))) p.Wgrad = EWgrad::BothInPlace;
            else if ((C % 256 == 0 || (C % 224 == 0 && bf16_dw && !accumulate)) && (wherever_served || C <= 8192)) p.Wgrad = EWgrad::GradInPlace;
        }
        return p;
    }
    std::vector<std::byte*> Live;

    Tensor temp_alloc(ETensorDType dtype, const std::vector<long>& shape) {
        Tensor t = Tensor::from_pointer(nullptr, Device, dtype, shape);
        const std::size_t need = (t.bytes() + 4095) / 4096 * 4096;
        if (Top + need > Capacity) throw std::runtime_error("QmmRunState: temporary stack exhausted");
        t.Data = Arena + Top;
        Top += need;
        if (Top > HighWater) HighWater = Top;
        Live.push_back(t.Data);
        return t;
    }
    void temp_free(Tensor& t) {
        if (Live.empty() || Live.back() != t.Data) throw std::logic_error("QmmRunState: temp_free out of LIFO order");
        Live.pop_back();
        Top = (std::size_t)(t.Data - Arena);
        t.Data = nullptr;
    }
    // Bytes of stack backward_qmm needs for one layer (the dry run of llama_run_state.cpp:362-390).
    static std::size_t backward_temp_bytes(int B, int T, int C, int OC, bool fuse_grad_transpose = false,
                                           DirectPlan plan = DirectPlan{}) {
        auto up = [](std::size_t b) { return (b + 4095) / 4096 * 4096; };
        const bool copies = plan.Wgrad == EWgrad::Copies;
        const std::size_t wt = plan.DgradInPlace ? 0 : up((std::size_t)C * OC);
        const std::size_t at = plan.Wgrad == EWgrad::BothInPlace ? 0 : up((std::size_t)C * B * T);
        const std::size_t gt = copies ? up((std::size_t)OC * B * T) : 0;
        if (fuse_grad_transpose) return gt + (wt > at ? wt : at);
        return wt > at + gt ? wt : at + gt;
    }
};

// out[B*T, OC] = inp[B*T, C] . weight[OC, C]^T (+ bias).  weight is already e4m3 with valid Stats.
inline void forward_qmm(Tensor& out, QuantizableTensor& inp, Tensor& weight, const Tensor& bias,
                        llmqBlasHandle_t handle, Tensor& workspace, int B, int T, int C, int OC,
                        const hipDeviceProp_t& dp, bool reuse_inp_quant, hipStream_t stream, EMatmulBackend backend) {
    if (weight.DType != ETensorDType::FP8_E4M3)
        throw std::invalid_argument("forward_qmm: this build implements the FP8 (e4m3 weight) branch only");
    if (!reuse_inp_quant) {
        quantize_with_abs_max(inp.Quant, inp.Quant.scale(), inp.Value, inp.Quant.abs_max(), (long)B * T * C, dp, stream);
    }
    matmul(out, weight, inp.Quant, bias, weight.scale(), inp.Quant.scale(), handle, workspace, OC, B * T, C,
           EMMTranspose::TN, false, stream, backend);
}

// dinp[B*T, C] = dout . weight ;  dweight[OC, C] (+)= dout^T . inp ;  dbias[OC] += column sums of dout when
// dbias is non-empty (bias_buffer: scratch of get_bias_backward_scratch_size bytes).  Argument order as in the
// reference (src/models/llama_model.cpp:280-285).
inline void backward_qmm(Tensor& dinp, Tensor& dweight, Tensor dbias, QuantizableTensor& dout, QuantizableTensor& inp,
                         Tensor& weight, Tensor bias_buffer, bool accumulate_gradient, QmmRunState& rs, int B, int T,
                         int C, int OC, bool reuse_inp, hipStream_t stream) {
    if (weight.DType != ETensorDType::FP8_E4M3)
        throw std::invalid_argument("backward_qmm: this build implements the FP8 (e4m3 weight) branch only");
    const QmmRunState::DirectPlan plan =
        rs.DirectGradLayout ? QmmRunState::direct_layout_plan(B, T, C, OC, dinp.DType, dweight.DType, accumulate_gradient,
                                                              rs.DirectGradLayoutWhereverServed)
                            : QmmRunState::DirectPlan{};
    const bool copies = plan.Wgrad == QmmRunState::EWgrad::Copies;
    Tensor grad_tp{};
    if (rs.FuseGradTranspose && copies) {
        grad_tp = rs.temp_alloc(dout.Quant.DType, {OC, (long)B * T});
        quantize_with_abs_max_and_transpose(dout.Quant, grad_tp, dout.Quant.scale(), dout.Value, dout.Quant.abs_max(),
                                            B * T, OC, rs.DeviceProp, stream);
    } else {
        quantize_with_abs_max(dout.Quant, dout.Quant.scale(), dout.Value, dout.Quant.abs_max(), (long)B * T * OC,
                              rs.DeviceProp, stream);
    }

    auto& inp_q = inp.Quant;
    Tensor no_bias{};
    if (plan.DgradInPlace) {
        // weight[OC, C] in its stored layout is the K-major first operand (mode NN): no transposed copy
        matmul(dinp, weight, dout.Quant, no_bias, weight.scale(), dout.Quant.scale(), rs.BlasHandle, rs.Workspace, C, B * T,
               OC, EMMTranspose::NN, false, stream, rs.MatmulBackend);
    } else {
        Tensor weight_tp = rs.temp_alloc(inp_q.DType, {C, OC});
        transpose(weight_tp, weight, OC, C, stream);
        matmul(dinp, weight_tp, dout.Quant, no_bias, weight.scale(), dout.Quant.scale(), rs.BlasHandle, rs.Workspace, C,
               B * T, OC, EMMTranspose::TN, false, stream, rs.MatmulBackend);
        rs.temp_free(weight_tp);
    }

    if (plan.Wgrad == QmmRunState::EWgrad::BothInPlace) {
        // activation [B*T, C] and gradient [B*T, OC] in their stored layouts are the two K-major operands (mode NT)
        if (!reuse_inp)
            quantize_with_abs_max(inp_q, inp_q.scale(), inp.Value, inp_q.abs_max(), (long)B * T * C, rs.DeviceProp, stream);
        matmul(dweight, inp_q, dout.Quant, no_bias, inp_q.scale(), dout.Quant.scale(), rs.BlasHandle, rs.Workspace, C, OC,
               B * T, EMMTranspose::NT, accumulate_gradient, stream, rs.MatmulBackend);
        if (!dbias.empty())
            backward_bias(dbias, dout.Quant, inp_q.scale(), dout.Quant.scale(), bias_buffer, B, T, OC, rs.DeviceProp, stream);
        return;
    }
    Tensor activation_tp = rs.temp_alloc(inp_q.DType, {C, (long)B * T});
    if (!rs.FuseGradTranspose && copies) grad_tp = rs.temp_alloc(dout.Quant.DType, {OC, (long)B * T});
    if (reuse_inp) {
        transpose(activation_tp, inp_q, B * T, C, stream);
    } else {
        // a stack temporary carries no Stats, so no scale is written here (llama_model.cpp:328)
        quantize_and_transpose_with_abs_max(activation_tp, activation_tp.scale(), inp.Value, inp.Quant.abs_max(),
                                            B * T, C, rs.DeviceProp, stream);
    }
    if (!copies) {
        // the quantized gradient in its stored layout [B*T, OC] is the K-major second operand (mode TT)
        matmul(dweight, activation_tp, dout.Quant, no_bias, inp_q.scale(), dout.Quant.scale(), rs.BlasHandle, rs.Workspace, C,
               OC, B * T, EMMTranspose::TT, accumulate_gradient, stream, rs.MatmulBackend);
    } else {
        if (!rs.FuseGradTranspose) transpose(grad_tp, dout.Quant, B * T, OC, stream);
        matmul(dweight, activation_tp, grad_tp, no_bias, inp_q.scale(), dout.Quant.scale(), rs.BlasHandle, rs.Workspace, C,
               OC, B * T, EMMTranspose::TN, accumulate_gradient, stream, rs.MatmulBackend);
    }
    if (!dbias.empty()) {
        backward_bias(dbias, dout.Quant, inp_q.scale(), dout.Quant.scale(), bias_buffer, B, T, OC, rs.DeviceProp, stream);
    }
    if (!copies) {
        rs.temp_free(activation_tp);
    } else if (rs.FuseGradTranspose) {
        rs.temp_free(activation_tp);
        rs.temp_free(grad_tp);
    } else {
        rs.temp_free(grad_tp);
        rs.temp_free(activation_tp);
    }
}

// ---- weight side: quantize on gather, cached per optimizer version ------------------------------------------
// The reference keeps bf16 master weights and hands the matmuls an e4m3 copy that it rebuilds only when the
// optimizer has changed the weights (src/models/llama_weights.cpp:207-223 convert_dtype_for_gather, :434-504 the
// LayerIdx / Version cache of LLamaWeightsManager).  On one GPU the gather itself is the identity; what remains is
// this cache: a small number of e4m3 slots (the reference double-buffers two layers), each remembering which layer
// and which weight version it holds.  The master tensor's Stats carry [abs_max, scale]: abs_max comes from the
// optimizer's epilogue (adamw_update) or from abs_max() at initialisation; the scale is written by the quantizer.
class QuantizedWeightCache {
public:
    struct Slot {
        Tensor Quant{};
        int LayerIdx = -1;
        int Version = -1;
    };

    // storage: one e4m3 tensor per slot, all of the weight's shape
    explicit QuantizedWeightCache(std::vector<Tensor> storage) {
        for (auto& t : storage) {
            if (t.DType != ETensorDType::FP8_E4M3) throw std::invalid_argument("QuantizedWeightCache: slots must be e4m3 tensors");
            Slots.push_back(Slot{t, -1, -1});
        }
        if (Slots.empty()) throw std::invalid_argument("QuantizedWeightCache: at least one slot");
    }

    // the optimizer has written new master weights: every cached copy is stale from now on
    void invalidate() { ++mVersion; }
    int version() const { return mVersion; }
    long quantize_calls() const { return mQuantizeCalls; }

    // e4m3 copy of layer `layer_idx`'s weight; requantized only if its slot holds another layer or an older version
    Tensor& get(int layer_idx, const Tensor& master, const hipDeviceProp_t& dp, hipStream_t stream) {
        Slot& s = Slots[(std::size_t)layer_idx % Slots.size()];
        if (master.nelem() != s.Quant.nelem()) throw std::invalid_argument("QuantizedWeightCache: shape mismatch");
        if (s.LayerIdx != layer_idx || s.Version != mVersion) {
            s.Quant.Stats = master.Stats;  // the copy shares the master's [abs_max, scale]
            quantize_with_abs_max(s.Quant, s.Quant.scale(), master, master.abs_max(), (long)master.nelem(), dp, stream);
            s.LayerIdx = layer_idx;
            s.Version = mVersion;
            ++mQuantizeCalls;
        }
        return s.Quant;
    }

private:
    std::vector<Slot> Slots;
    int mVersion = 0;
    long mQuantizeCalls = 0;
};

#endif  // LLMQ_QMM_HPP

// C++ host side of the MoE layer over the C ABI of libomega_hip.so, mirroring the reference's Java Layer
// contract (the reference is Java; this build has no JDK, so the compiled-language mirror is C++).
//
//   omega::Tensor    the fields of J/engine/tensor/Tensor.java:23-47 the path uses: number/channel/height/width,
//                    host float data, a device address, hostToDevice()/syncHost() (Tensor.java:559-579)
//   omega::Layer     the abstract methods of J/engine/nn/layer/Layer.java:66-104
//   omega::MoELayer  constructor in the house style of LlamaMLPLayer(embedDim, nChannel, multiple_of, bias, network)
//                    (J/engine/nn/layer/llama/LlamaMLPLayer.java:47-63) with the explicit hidden size of DiTSwiGLUFFN;
//                    forward(Tensor) = setInput -> init -> output (LlamaMLPLayer.java:200-217);
//                    saveModel/loadModel write raw little-endian float32 in the order gate, (gate bias), then
//                    w1,w3,w2 per expert (routed, then shared), as LlamaMLPLayer.java:273-283 does for one MLP;
//                    a failing library call throws std::runtime_error("Error code N:msg"), the checkCUDA style
//                    (J/engine/gpu/CUDAMemoryManager.java:179-201); back(Tensor) = initBack -> setDelta -> diff
//                    (LlamaMLPLayer.java:186-199), update()/accGrad() as FullyLayer.java:569-607, the AdamW branch
//                    and the layer's part of Network.clipGradNorm beside them.
// Host tensors are fp32 like the reference's; a bf16 layer converts on the device at the boundary.
#pragma once
#include <cstdint>
#include <cstdio>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "omega_hip.h"

namespace omega {

inline void check(omega_ctx *ctx, int st)
{
    if (st != OMEGA_OK) {
        const char *msg = omega_hip_last_error(ctx);
        throw std::runtime_error(msg && *msg ? msg : "Error code " + std::to_string(st));
    }
}

// One device + one stream (replaces CUDAManager / CUDAPool for this path).
class Context {
public:
    explicit Context(int device = 0)
    {
        int st = omega_hip_ctx_create(device, &ctx_);
        if (st != OMEGA_OK) throw std::runtime_error(omega_hip_last_error(nullptr));
    }
    ~Context() { omega_hip_ctx_destroy(ctx_); }
    Context(const Context &) = delete;
    Context &operator=(const Context &) = delete;
    omega_ctx *get() const { return ctx_; }
    void sync() { check(ctx_, omega_hip_sync(ctx_)); }

private:
    omega_ctx *ctx_ = nullptr;
};

struct Tensor {
    int number = 0, channel = 0, height = 0, width = 0;
    std::vector<float> data;   // host copy (fp32)
    void *gpuData = nullptr;   // device address, fp32 [number*channel*height*width]
    Context *ctx = nullptr;

    Tensor() = default;
    Tensor(int n, int c, int h, int w, Context *cx, bool hasGPU = true) : number(n), channel(c), height(h), width(w), ctx(cx)
    {
        data.assign((size_t)n * c * h * w, 0.0f);
        if (hasGPU) check(ctx->get(), omega_hip_malloc(ctx->get(), data.size() * 4, &gpuData));
    }
    Tensor(const Tensor &) = delete;
    Tensor &operator=(const Tensor &) = delete;
    ~Tensor()
    {
        if (gpuData) omega_hip_free(ctx->get(), gpuData);
    }
    size_t dataLength() const { return data.size(); }
    bool isHasGPU() const { return gpuData != nullptr; }
    void hostToDevice() { check(ctx->get(), omega_hip_memcpy_h2d(ctx->get(), gpuData, data.data(), data.size() * 4)); }
    void syncHost() { check(ctx->get(), omega_hip_memcpy_d2h(ctx->get(), data.data(), gpuData, data.size() * 4)); }
};

class Layer {
public:
    virtual ~Layer() = default;
    int number = 0, channel = 0, height = 0, width = 0, oChannel = 0, oHeight = 0, oWidth = 0;
    Tensor *input = nullptr;
    virtual void init() = 0;
    virtual void initBack() = 0;
    virtual void initParam() = 0;
    virtual void output() = 0;
    virtual Tensor *getOutput() = 0;
    virtual void diff() = 0;
    virtual void forward() = 0;
    virtual void back() = 0;
    virtual void backTemp() = 0;
    virtual void forward(Tensor &input) = 0;
    virtual void back(Tensor &delta) = 0;
    virtual void update() = 0;
    virtual void accGrad(float scale) = 0;
    virtual void showDiff() = 0;
    virtual const char *getLayerType() const = 0;
    virtual const float *output(const float *input) = 0;  // the legacy host-array path: float[][][][] output(float[][][][])
    virtual void initCache() = 0;
    void setInput(Tensor &in) { input = &in; }
};

class MoELayer : public Layer {
public:
    MoELayer(int embedDim, int hidden, int nExperts, int topK, bool renorm, int nShared, bool bias, Context &ctx,
             int dtype = OMEGA_DTYPE_F32, int routerMode = OMEGA_ROUTER_EXACT)
        : ctx_(ctx), embedDim_(embedDim), hidden_(hidden), nExperts_(nExperts), topK_(topK), nShared_(nShared), bias_(bias),
          dtype_(dtype)
    {
        oChannel = 1;
        oHeight = 1;
        oWidth = embedDim;
        omega_moe_config cfg{0, embedDim, nExperts, topK, hidden, nShared, renorm ? 1 : 0, bias ? 1 : 0, dtype, routerMode};
        check(ctx_.get(), omega_moe_create(ctx_.get(), &cfg, &moe_));
    }
    ~MoELayer() override
    {
        omega_moe_destroy(moe_);
        void *low[] = {xLow_, outLow_, deltaLow_, diffLow_};
        for (void *p : low)
            if (p) omega_hip_free(ctx_.get(), p);
    }

    // parameters arrive as fp32 host arrays in the reference's [out,in] layout
    void setGate(const float *Wg, const float *bg = nullptr)
    {
        upload(OMEGA_W_GATE, 0, Wg, (size_t)nExperts_ * embedDim_);
        if (bg) check(ctx_.get(), omega_moe_set_weights(moe_, OMEGA_W_GATE_BIAS, 0, bg, 0));
    }
    // weight of the RMSNorm in front of the layer (norm2 of the block), fp32
    void setNorm(const float *gamma) { check(ctx_.get(), omega_moe_set_weights(moe_, OMEGA_W_NORM, 0, gamma, 0)); }
    void setExpert(int g, const float *W1, const float *W3, const float *W2)
    {
        const size_t n = (size_t)hidden_ * embedDim_;
        upload(OMEGA_W_W1, g, W1, n);
        upload(OMEGA_W_W3, g, W3, n);
        upload(OMEGA_W_W2, g, W2, n);
    }

    // RandomUtils.setSeed(seed) + the house-style initialisation of LlamaMLPLayer.initLayers
    // (J/engine/nn/layer/llama/LlamaMLPLayer.java:68-90): every weight normal_(n, 0.01f, 0.02f) from ONE java.util.Random
    // (J/common/utils/RandomUtils.java:18-28,697-703); the gate first (the reference has none: drawn like the others),
    // then per expert linear1 (W1), linear2 (W2), linear3 (W3) in the order the reference constructs them
    void initJava(int64_t seed, float mean = 0.01f, float std = 0.02f)
    {
        omega_jrandom r;
        omega_jrandom_seed(&r, seed);
        const size_t n = (size_t)hidden_ * embedDim_;
        std::vector<float> wg((size_t)nExperts_ * embedDim_), w1(n), w2(n), w3(n);
        omega_jrandom_normal(&r, wg.data(), wg.size(), mean, std);
        setGate(wg.data());
        for (int g = 0; g < nExperts_ + nShared_; ++g) {
            omega_jrandom_normal(&r, w1.data(), n, mean, std);
            omega_jrandom_normal(&r, w2.data(), n, mean, std);
            omega_jrandom_normal(&r, w3.data(), n, mean, std);
            setExpert(g, w1.data(), w3.data(), w2.data());
        }
    }

    void init() override
    {
        number = input->number;
        if (!output_ || output_->number != number) {
            output_.reset(new Tensor(number, oChannel, oHeight, oWidth, &ctx_, true));
            if (dtype_ == OMEGA_DTYPE_BF16) {
                if (xLow_) omega_hip_free(ctx_.get(), xLow_);
                if (outLow_) omega_hip_free(ctx_.get(), outLow_);
                check(ctx_.get(), omega_hip_malloc(ctx_.get(), (size_t)number * embedDim_ * 2, &xLow_));
                check(ctx_.get(), omega_hip_malloc(ctx_.get(), (size_t)number * embedDim_ * 2, &outLow_));
            }
        }
    }
    // (re)allocates the input gradient when the batch size changes (FullyLayer.initBack,
    // J/engine/nn/layer/FullyLayer.java:130-144); the parameter gradients live in the native handle
    void initBack() override
    {
        if (!diff_ || diff_->number != number) {
            diff_.reset(new Tensor(number, oChannel, oHeight, oWidth, &ctx_, true));
            if (dtype_ == OMEGA_DTYPE_BF16) {
                if (deltaLow_) omega_hip_free(ctx_.get(), deltaLow_);
                if (diffLow_) omega_hip_free(ctx_.get(), diffLow_);
                check(ctx_.get(), omega_hip_malloc(ctx_.get(), (size_t)number * embedDim_ * 2, &deltaLow_));
                check(ctx_.get(), omega_hip_malloc(ctx_.get(), (size_t)number * embedDim_ * 2, &diffLow_));
            }
        }
    }
    void initParam() override {}
    void output() override { run(false); }
    // second half of the transformer block in one call: output = input + layer(rmsnorm(input))
    // (getNorm2().forward(tmp1); getMlp().forward(...); Tensor_OP().add(mlp out, tmp1, tmp2),
    //  J/engine/nn/layer/llama/LlamaTransformerBlock.java:134-136); setNorm must have been called
    void forwardBlock(Tensor &in)
    {
        if (in.width != embedDim_ || !in.isHasGPU()) throw std::runtime_error("Error code 1:input width does not match embedDim or tensor has no device data");
        setInput(in);
        init();
        run(true);
    }
    Tensor *getOutput() override { return output_.get(); }
    void forward() override
    {
        init();
        output();
    }
    void forward(Tensor &in) override
    {
        if (in.width != embedDim_ || !in.isHasGPU()) throw std::runtime_error("Error code 1:input width does not match embedDim or tensor has no device data");
        setInput(in);
        init();
        output();
    }
    // back(Tensor delta) = initBack -> setDelta -> diff (LlamaMLPLayer.back, J/engine/nn/layer/llama/LlamaMLPLayer.java:186-199);
    // must follow forward(Tensor) of the same input.  The input gradient is getDiff(); the parameter gradients are
    // overwritten inside the handle (grad()).
    void back(Tensor &delta) override
    {
        if (!input || !output_) throw std::runtime_error("Error code 1:back without a forward");
        if (delta.number != number || delta.width != embedDim_ || !delta.isHasGPU())
            throw std::runtime_error("Error code 1:delta shape does not match the output or tensor has no device data");
        initBack();
        delta_ = &delta;
        diff();
    }
    void back() override
    {
        if (!delta_) throw std::runtime_error("Error code 1:back() without a delta");
        initBack();
        diff();
    }
    // backward of forwardBlock: getMlp().back(delta); getNorm2().back(getMlp().diff); add(norm2.diff, delta)
    // (J/engine/nn/layer/llama/LlamaTransformerBlock.java:156-158); getDiff() is the gradient of the block's input,
    // grad(OMEGA_W_NORM) the gradient of the norm weight
    void backBlock(Tensor &delta)
    {
        if (!input || !output_) throw std::runtime_error("Error code 1:back without a forward");
        if (delta.number != number || delta.width != embedDim_ || !delta.isHasGPU())
            throw std::runtime_error("Error code 1:delta shape does not match the output or tensor has no device data");
        initBack();
        delta_ = &delta;
        runBack(true);
    }
    void diff() override { runBack(false); }
    // the hooks LlamaMLPLayer leaves empty (J/engine/nn/layer/llama/LlamaMLPLayer.java:247-271): nothing to show, no
    // legacy host-array path (it returns null there), no cache, no temporary backward
    void backTemp() override {}
    void showDiff() override {}
    const float *output(const float *) override { return nullptr; }
    void initCache() override {}
    void runBack(bool block)
    {
        const size_t n = (size_t)number * embedDim_;
        auto bwd = block ? omega_moe_backward_block : omega_moe_backward;
        if (dtype_ == OMEGA_DTYPE_BF16) {
            // xLow_ still holds the input of the forward call
            check(ctx_.get(), omega_hip_convert(ctx_.get(), deltaLow_, OMEGA_DTYPE_BF16, delta_->gpuData, OMEGA_DTYPE_F32, n));
            check(ctx_.get(), bwd(moe_, xLow_, deltaLow_, number, diffLow_));
            check(ctx_.get(), omega_hip_convert(ctx_.get(), diff_->gpuData, OMEGA_DTYPE_F32, diffLow_, OMEGA_DTYPE_BF16, n));
        } else {
            check(ctx_.get(), bwd(moe_, input->gpuData, delta_->gpuData, number, diff_->gpuData));
        }
    }
    Tensor *getDiff() { return diff_.get(); }
    // forward keeps h1 / h3 for back(), as the reference's layers keep their outputs
    void setTraining(bool on) { check(ctx_.get(), omega_moe_set_training(moe_, on ? 1 : 0)); }
    /// OMEGA_GATHER_AUTO / _COPY / _ON_LOAD: how the rows of x reach the experts of a bf16 layer
    void setGatherMode(int mode) { check(ctx_.get(), omega_moe_set_gather_mode(moe_, mode)); }
    bool gatherOnLoad() const { return omega_moe_gather_on_load(moe_) != 0; }
    // update() of a layer without an updater: w -= learnRate * diffW (FullyLayer.update, FullyLayer.java:569-590)
    float learnRate = 0.0f;
    bool freeze = false;  // Layer.freeze: a frozen layer's update() does nothing (FullyLayer.java:571)
    void update() override
    {
        if (!freeze) check(ctx_.get(), omega_moe_update(moe_, learnRate));
    }
    // update() under the AdamW updater (AdamW.update, AdamW.java:69-92): trainTime is network.train_time, from 1
    void updateAdamW(float lr, int trainTime, float beta1 = 0.9f, float beta2 = 0.95f, float weightDecay = 1e-4f)
    {
        if (freeze) return;
        check(ctx_.get(), omega_moe_update_adamw(moe_, lr, beta1, beta2, weightDecay, trainTime));
    }
    void accGrad(float scale) override { check(ctx_.get(), omega_moe_acc_grad(moe_, scale)); }
    // the layer's part of Network.clipGradNorm (Network.java:379-432): its term of the total, and the scaling
    float gradSumSq()
    {
        float v = 0.0f;
        check(ctx_.get(), omega_moe_grad_sumsq(moe_, &v));
        return v;
    }
    void scaleGrad(float coef) { check(ctx_.get(), omega_moe_scale_grad(moe_, coef)); }
    // one parameter gradient (fp32, layout of its weight): OMEGA_W_GATE, OMEGA_W_GATE_BIAS, OMEGA_W_W1 / W3 / W2 of expert g
    std::vector<float> grad(int which, int g = 0)
    {
        const size_t n = which == OMEGA_W_GATE        ? (size_t)nExperts_ * embedDim_
                         : which == OMEGA_W_GATE_BIAS ? (size_t)nExperts_
                         : which == OMEGA_W_NORM      ? (size_t)embedDim_
                                                      : (size_t)hidden_ * embedDim_;
        std::vector<float> h(n);
        check(ctx_.get(), omega_moe_get_grad(moe_, which, g, h.data(), 0));
        return h;
    }
    const char *getLayerType() const override { return "feed_forward"; }

    void getRouting(std::vector<int32_t> &ids, std::vector<float> &w, std::vector<int32_t> &counts)
    {
        ids.resize((size_t)number * topK_);
        w.resize(ids.size());
        counts.resize(nExperts_);
        check(ctx_.get(), omega_moe_get_routing(moe_, number, ids.data(), w.data(), counts.data(), nullptr, nullptr, nullptr));
    }

    // the block form's parameters in the order LlamaTransformerBlock.saveModel writes them for its FFN half: norm2
    // (RMSLayer.saveModel: gamma), then the mlp (J/engine/nn/layer/llama/LlamaTransformerBlock.java:263-275)
    void saveModelBlock(FILE *f)
    {
        std::vector<float> g(embedDim_);
        check(ctx_.get(), omega_moe_get_weights(moe_, OMEGA_W_NORM, 0, g.data(), 0));
        if (fwrite(g.data(), 4, g.size(), f) != g.size()) throw std::runtime_error("Error code 1:short write");
        saveModel(f);
    }
    void loadModelBlock(FILE *f)
    {
        std::vector<float> g(embedDim_);
        if (fread(g.data(), 4, g.size(), f) != g.size()) throw std::runtime_error("Error code 1:checkpoint ends early");
        setNorm(g.data());
        loadModel(f);
    }
    void saveModel(FILE *f) { eachParam([&](int which, int g, size_t n) { std::vector<float> h = download(which, g, n); if (fwrite(h.data(), 4, n, f) != n) throw std::runtime_error("Error code 1:short write"); }); }
    void loadModel(FILE *f) { eachParam([&](int which, int g, size_t n) { std::vector<float> h(n); if (fread(h.data(), 4, n, f) != n) throw std::runtime_error("Error code 1:checkpoint ends early"); if (which == OMEGA_W_GATE_BIAS) check(ctx_.get(), omega_moe_set_weights(moe_, which, g, h.data(), 0)); else upload(which, g, h.data(), n); }); }

private:
    void run(bool block)
    {
        const size_t n = (size_t)number * embedDim_;
        auto fwd = block ? omega_moe_forward_block : omega_moe_forward;
        if (dtype_ == OMEGA_DTYPE_BF16) {
            check(ctx_.get(), omega_hip_convert(ctx_.get(), xLow_, OMEGA_DTYPE_BF16, input->gpuData, OMEGA_DTYPE_F32, n));
            check(ctx_.get(), fwd(moe_, xLow_, number, outLow_));
            check(ctx_.get(), omega_hip_convert(ctx_.get(), output_->gpuData, OMEGA_DTYPE_F32, outLow_, OMEGA_DTYPE_BF16, n));
        } else {
            check(ctx_.get(), fwd(moe_, input->gpuData, number, output_->gpuData));
        }
    }
    template <class F> void eachParam(F f)
    {
        f(OMEGA_W_GATE, 0, (size_t)nExperts_ * embedDim_);
        if (bias_) f(OMEGA_W_GATE_BIAS, 0, (size_t)nExperts_);
        for (int g = 0; g < nExperts_ + nShared_; ++g) {
            f(OMEGA_W_W1, g, (size_t)hidden_ * embedDim_);
            f(OMEGA_W_W3, g, (size_t)hidden_ * embedDim_);
            f(OMEGA_W_W2, g, (size_t)hidden_ * embedDim_);
        }
    }
    // fp32 host array -> layer dtype on the device -> layer storage
    void upload(int which, int g, const float *h, size_t n)
    {
        if (dtype_ == OMEGA_DTYPE_F32) {
            check(ctx_.get(), omega_moe_set_weights(moe_, which, g, h, 0));
            return;
        }
        void *f32 = nullptr, *low = nullptr;
        check(ctx_.get(), omega_hip_malloc(ctx_.get(), n * 4, &f32));
        check(ctx_.get(), omega_hip_malloc(ctx_.get(), n * 2, &low));
        int st = omega_hip_memcpy_h2d(ctx_.get(), f32, h, n * 4);
        if (st == OMEGA_OK) st = omega_hip_convert(ctx_.get(), low, OMEGA_DTYPE_BF16, f32, OMEGA_DTYPE_F32, n);
        if (st == OMEGA_OK) st = omega_moe_set_weights(moe_, which, g, low, 1);
        omega_hip_free(ctx_.get(), f32);
        omega_hip_free(ctx_.get(), low);
        check(ctx_.get(), st);
    }
    std::vector<float> download(int which, int g, size_t n)
    {
        std::vector<float> h(n);
        if (dtype_ == OMEGA_DTYPE_F32 || which == OMEGA_W_GATE_BIAS) {
            check(ctx_.get(), omega_moe_get_weights(moe_, which, g, h.data(), 0));
            return h;
        }
        void *f32 = nullptr, *low = nullptr;
        check(ctx_.get(), omega_hip_malloc(ctx_.get(), n * 4, &f32));
        check(ctx_.get(), omega_hip_malloc(ctx_.get(), n * 2, &low));
        int st = omega_moe_get_weights(moe_, which, g, low, 1);
        if (st == OMEGA_OK) st = omega_hip_convert(ctx_.get(), f32, OMEGA_DTYPE_F32, low, OMEGA_DTYPE_BF16, n);
        if (st == OMEGA_OK) st = omega_hip_memcpy_d2h(ctx_.get(), h.data(), f32, n * 4);
        omega_hip_free(ctx_.get(), f32);
        omega_hip_free(ctx_.get(), low);
        check(ctx_.get(), st);
        return h;
    }

    Context &ctx_;
    omega_moe *moe_ = nullptr;
    int embedDim_, hidden_, nExperts_, topK_, nShared_;
    bool bias_;
    int dtype_;
    std::unique_ptr<Tensor> output_, diff_;
    Tensor *delta_ = nullptr;
    void *xLow_ = nullptr, *outLow_ = nullptr, *deltaLow_ = nullptr, *diffLow_ = nullptr;
};

}  // namespace omega

/*
 * NOT COMPILED BY THIS BUILD: neither the build image nor the GPU machines have a JDK.  This is the layer a
 * maintainer adds to Omega-AI (src/main/java/com/omega/engine/nn/layer/moe/MoELayer.java, JDK >= 22); every native
 * call and its order mirror the compiled and GPU-tested C++ twin, omega-ai_amd/host/MoELayer.hpp, method for method.
 */
package com.omega.engine.nn.layer.moe;

import java.io.IOException;
import java.io.RandomAccessFile;
import java.lang.foreign.MemorySegment;
import java.nio.ByteBuffer;
import java.nio.ByteOrder;

import com.omega.engine.gpu.hip.OmegaHip;
import com.omega.engine.nn.layer.Layer;
import com.omega.engine.nn.layer.LayerType;
import com.omega.engine.nn.network.Network;
import com.omega.engine.parallel.ddp.distributed.SerializablePointer;
import com.omega.engine.tensor.Tensor;
import com.omega.engine.updater.AdamW;
import com.omega.engine.updater.UpdaterFactory;

/**
 * Mixture-of-experts FFN layer for the FFN slot of a transformer block
 * (LlamaTransformerBlock.java:97,135: getMlp().forward(getNorm2().getOutput())).  Constructor in the house style of
 * LlamaMLPLayer(embedDim, nChannel, multiple_of, bias, network) (LlamaMLPLayer.java:47-63) with the explicit hidden size
 * of DiTSwiGLUFFN.  The layer owns its weights inside the native handle and never touches JCuda: host tensors use the
 * CPU constructor Tensor(number, channel, height, width, float[]) (Tensor.java:114-122), device addresses are exposed as
 * SerializablePointer(long) (SerializablePointer.java:16-18), and all transfers go through libomega_hip.so.  It
 * tolerates network == null (no Network can be constructed on a host without libcuda, Network.java:85-92).
 */
public class MoELayer extends Layer {
    private final int embedDim, hidden, nExperts, topK, nShared;
    private final boolean renorm, gateBias;
    private final int dtype;                       // OmegaHip.F32 or OmegaHip.BF16: storage type inside the layer
    private final MemorySegment ctx, moe;
    // fp32 device copies of the host tensors (input, output, delta, diff) and, for bf16 layers, their bf16 twins
    private long xDev, outDev, deltaDev, diffDev, xLow, outLow, deltaLow, diffLow;
    private int devRows, devRowsBack;
    /** Parameters of the AdamW updater when the network uses it (AdamWKernel.java:25-26). */
    public float beta1 = 0.9f, beta2 = 0.95f;

    public MoELayer(int embedDim, int hidden, int nExperts, int topK, boolean renorm, int nShared, boolean bias, Network network) {
        this(embedDim, hidden, nExperts, topK, renorm, nShared, bias, network, OmegaHip.F32, OmegaHip.ROUTER_EXACT);
    }

    public MoELayer(int embedDim, int hidden, int nExperts, int topK, boolean renorm, int nShared, boolean bias, Network network,
                    int dtype, int routerMode) {
        this.network = network;                    // may be null on an AMD host
        this.embedDim = embedDim;
        this.hidden = hidden;
        this.nExperts = nExperts;
        this.topK = topK;
        this.renorm = renorm;
        this.nShared = nShared;
        this.gateBias = bias;
        this.dtype = dtype;
        this.channel = 1;
        this.height = 1;
        this.width = embedDim;
        this.oChannel = 1;                         // LlamaMLPLayer.java:56-58
        this.oHeight = 1;
        this.oWidth = embedDim;
        this.hasBias = bias;
        this.hasParams = true;
        this.ctx = OmegaHip.ctxCreate(0);
        this.moe = OmegaHip.moeCreate(ctx, 0, embedDim, nExperts, topK, hidden, nShared, renorm, bias, dtype, routerMode);
        if (network != null) {                     // FullyLayer.java:57-70
            network.paramLayers.add(this);
            this.setUpdater(UpdaterFactory.create(network));
        }
    }

    /** Releases the native handle and the device buffers (the reference frees through CUDAMemoryManager.free). */
    public void close() {
        OmegaHip.moeDestroy(moe);
        for (long p : new long[]{xDev, outDev, deltaDev, diffDev, xLow, outLow, deltaLow, diffLow}) {
            OmegaHip.free(ctx, p);
        }
        OmegaHip.ctxDestroy(ctx);
    }

    // ---- parameters: fp32 host arrays in the reference's [out,in] layout (FullyLayer.java:181) ----

    private void upload(int which, int g, float[] h) {
        if (dtype == OmegaHip.F32 || which == OmegaHip.W_GATE_BIAS || which == OmegaHip.W_NORM) {
            OmegaHip.setWeightsHost(ctx, moe, which, g, h);
            return;
        }
        long f32 = OmegaHip.malloc(ctx, 4L * h.length), low = OmegaHip.malloc(ctx, 2L * h.length);
        try {
            OmegaHip.h2d(ctx, f32, h, h.length);
            OmegaHip.convert(ctx, low, OmegaHip.BF16, f32, OmegaHip.F32, h.length);
            OmegaHip.setWeightsDevice(ctx, moe, which, g, low);
        } finally {
            OmegaHip.free(ctx, f32);
            OmegaHip.free(ctx, low);
        }
    }

    private float[] download(int which, int g, int n) {
        float[] h = new float[n];
        if (dtype == OmegaHip.F32 || which == OmegaHip.W_GATE_BIAS || which == OmegaHip.W_NORM) {
            OmegaHip.getWeightsHost(ctx, moe, which, g, h);
            return h;
        }
        long f32 = OmegaHip.malloc(ctx, 4L * n), low = OmegaHip.malloc(ctx, 2L * n);
        try {
            OmegaHip.getWeightsDevice(ctx, moe, which, g, low);
            OmegaHip.convert(ctx, f32, OmegaHip.F32, low, OmegaHip.BF16, n);
            OmegaHip.d2h(ctx, h, f32, n);
        } finally {
            OmegaHip.free(ctx, f32);
            OmegaHip.free(ctx, low);
        }
        return h;
    }

    public void setGate(float[] wg, float[] bg) {
        upload(OmegaHip.W_GATE, 0, wg);
        if (bg != null) {
            upload(OmegaHip.W_GATE_BIAS, 0, bg);
        }
    }

    /** Weight of the RMSNorm in front of the layer (norm2 of the block), used by forwardBlock. */
    public void setNorm(float[] gamma) {
        upload(OmegaHip.W_NORM, 0, gamma);
    }

    public void setExpert(int g, float[] w1, float[] w3, float[] w2) {
        upload(OmegaHip.W_W1, g, w1);
        upload(OmegaHip.W_W3, g, w3);
        upload(OmegaHip.W_W2, g, w2);
    }

    /** House-style initialisation (LlamaMLPLayer.java:68-90): every weight RandomUtils.normal_(n, 0.01f, 0.02f); the gate
     *  first, then per expert linear1 (w1), linear2 (w2), linear3 (w3) in the order the reference constructs them. */
    @Override
    public void initParam() {
        int n = hidden * embedDim;
        setGate(com.omega.common.utils.RandomUtils.normal_(nExperts * embedDim, 0.01f, 0.02f), null);
        for (int g = 0; g < nExperts + nShared; g++) {
            float[] w1 = com.omega.common.utils.RandomUtils.normal_(n, 0.01f, 0.02f);
            float[] w2 = com.omega.common.utils.RandomUtils.normal_(n, 0.01f, 0.02f);
            float[] w3 = com.omega.common.utils.RandomUtils.normal_(n, 0.01f, 0.02f);
            setExpert(g, w1, w3, w2);
        }
    }

    // ---- forward ----

    @Override
    public void init() {                           // LlamaMLPLayer.java:98-104
        this.number = this.input.number;
        if (this.output == null || this.output.number != this.number) {
            this.output = new Tensor(number, oChannel, oHeight, oWidth, new float[number * oWidth]);   // CPU ctor, no JCuda
        }
        if (devRows != number) {
            for (long p : new long[]{xDev, outDev, xLow, outLow}) {
                OmegaHip.free(ctx, p);
            }
            long n = (long) number * embedDim;
            xDev = OmegaHip.malloc(ctx, 4 * n);
            outDev = OmegaHip.malloc(ctx, 4 * n);
            xLow = outLow = 0L;
            if (dtype == OmegaHip.BF16) {
                xLow = OmegaHip.malloc(ctx, 2 * n);
                outLow = OmegaHip.malloc(ctx, 2 * n);
            }
            devRows = number;
            this.output.setHasGPU(true);           // Tensor.java:555-557,704-706
            this.output.setGpuData(new SerializablePointer(outDev));
        }
    }

    private void run(boolean block) {
        int n = number * embedDim;
        OmegaHip.h2d(ctx, xDev, input.data, n);
        if (dtype == OmegaHip.BF16) {
            OmegaHip.convert(ctx, xLow, OmegaHip.BF16, xDev, OmegaHip.F32, n);
            OmegaHip.forward(ctx, moe, xLow, number, outLow, block);
            OmegaHip.convert(ctx, outDev, OmegaHip.F32, outLow, OmegaHip.BF16, n);
        } else {
            OmegaHip.forward(ctx, moe, xDev, number, outDev, block);
        }
        OmegaHip.d2h(ctx, output.data, outDev, n);     // fills output.data itself instead of relying on syncHost()
    }

    @Override
    public void output() {
        run(false);
    }

    @Override
    public void forward() {
        this.init();
        this.output();
    }

    @Override
    public void forward(Tensor input) {            // LlamaMLPLayer.java:200-217
        if (input.width != embedDim) {
            throw new RuntimeException("Error code 1:input width does not match embedDim");
        }
        this.setInput(input);
        this.init();
        this.output();
    }

    /** Second half of the transformer block in one call: output = input + layer(rmsnorm(input))
     *  (getNorm2().forward(tmp1); getMlp().forward(...); Tensor_OP().add(mlp out, tmp1, tmp2),
     *  LlamaTransformerBlock.java:134-136); setNorm must have been called. */
    public void forwardBlock(Tensor input) {
        if (input.width != embedDim) {
            throw new RuntimeException("Error code 1:input width does not match embedDim");
        }
        this.setInput(input);
        this.init();
        run(true);
    }

    @Override
    public Tensor getOutput() {
        return output;
    }

    @Override
    public LayerType getLayerType() {
        return LayerType.feed_forward;
    }

    /** The legacy host-array path returns null in LlamaMLPLayer too (LlamaMLPLayer.java:247-271). */
    @Override
    public float[][][][] output(float[][][][] input) {
        return null;
    }

    @Override
    public void initCache() {
    }

    @Override
    public void backTemp() {
    }

    @Override
    public void showDiff() {
    }

    // ---- backward ----

    @Override
    public void initBack() {                       // FullyLayer.java:130-144
        if (this.diff == null || this.diff.number != this.number) {
            this.diff = new Tensor(number, oChannel, oHeight, oWidth, new float[number * oWidth]);
        }
        if (devRowsBack != number) {
            for (long p : new long[]{deltaDev, diffDev, deltaLow, diffLow}) {
                OmegaHip.free(ctx, p);
            }
            long n = (long) number * embedDim;
            deltaDev = OmegaHip.malloc(ctx, 4 * n);
            diffDev = OmegaHip.malloc(ctx, 4 * n);
            deltaLow = diffLow = 0L;
            if (dtype == OmegaHip.BF16) {
                deltaLow = OmegaHip.malloc(ctx, 2 * n);
                diffLow = OmegaHip.malloc(ctx, 2 * n);
            }
            devRowsBack = number;
            this.diff.setHasGPU(true);
            this.diff.setGpuData(new SerializablePointer(diffDev));
        }
    }

    private void runBack(boolean block) {
        int n = number * embedDim;
        OmegaHip.h2d(ctx, deltaDev, delta.data, n);
        if (dtype == OmegaHip.BF16) {              // xLow still holds the input of the forward call
            OmegaHip.convert(ctx, deltaLow, OmegaHip.BF16, deltaDev, OmegaHip.F32, n);
            OmegaHip.backward(ctx, moe, xLow, deltaLow, number, diffLow, block);
            OmegaHip.convert(ctx, diffDev, OmegaHip.F32, diffLow, OmegaHip.BF16, n);
        } else {
            OmegaHip.backward(ctx, moe, xDev, deltaDev, number, diffDev, block);
        }
        OmegaHip.d2h(ctx, diff.data, diffDev, n);
    }

    @Override
    public void diff() {
        runBack(false);
    }

    @Override
    public void back() {
        if (this.delta == null) {
            throw new RuntimeException("Error code 1:back() without a delta");
        }
        this.initBack();
        this.diff();
    }

    @Override
    public void back(Tensor delta) {               // LlamaMLPLayer.java:186-199: initBack -> setDelta -> diff
        if (this.input == null || this.output == null) {
            throw new RuntimeException("Error code 1:back without a forward");
        }
        if (delta.number != number || delta.width != embedDim) {
            throw new RuntimeException("Error code 1:delta shape does not match the output");
        }
        this.initBack();
        this.delta = delta;
        this.diff();
    }

    /** Backward of forwardBlock: getMlp().back(delta); getNorm2().back(getMlp().diff); add(norm2.diff, delta)
     *  (LlamaTransformerBlock.java:156-158); diff is the gradient of the block's input, grad(W_NORM, 0) the norm weight's. */
    public void backBlock(Tensor delta) {
        if (this.input == null || this.output == null) {
            throw new RuntimeException("Error code 1:back without a forward");
        }
        if (delta.number != number || delta.width != embedDim) {
            throw new RuntimeException("Error code 1:delta shape does not match the output");
        }
        this.initBack();
        this.delta = delta;
        runBack(true);
    }

    /** Forward keeps h1 / h3 for back(), as the reference's layers keep their outputs. */
    public void setTraining(boolean on) {
        OmegaHip.setTraining(ctx, moe, on);
    }

    /** How the rows of x reach the experts of a bf16 layer: 0 by shape, 1 gathered copy, 2 fetched by the up product's loads. */
    public void setGatherMode(int mode) {
        OmegaHip.setGatherMode(ctx, moe, mode);
    }

    /** One parameter gradient (fp32, layout of its weight): W_GATE, W_GATE_BIAS, W_NORM, W_W1 / W_W3 / W_W2 of expert g. */
    public float[] grad(int which, int g) {
        int n = which == OmegaHip.W_GATE ? nExperts * embedDim
                : which == OmegaHip.W_GATE_BIAS ? nExperts
                : which == OmegaHip.W_NORM ? embedDim : hidden * embedDim;
        float[] h = new float[n];
        OmegaHip.getGradHost(ctx, moe, which, g, h);
        return h;
    }

    @Override
    public void accGrad(float scale) {             // FullyLayer.java:593-607
        OmegaHip.accGrad(ctx, moe, scale);
    }

    @Override
    public void update() {                         // FullyLayer.java:569-590
        if (this.freeze) {
            return;
        }
        if (this.updater == null) {
            OmegaHip.update(ctx, moe, this.learnRate);
        } else if (this.updater instanceof AdamW) {    // AdamW.update, AdamW.java:69-92: layer.learnRate = network.learnRate
            this.learnRate = network.learnRate;
            OmegaHip.updateAdamW(ctx, moe, this.learnRate, beta1, beta2, network.weight_decay, network.train_time);
        } else {
            throw new UnsupportedOperationException("MoELayer: only the plain update and AdamW are built into libomega_hip.so");
        }
    }

    /** The layer's term of Network.clipGradNorm's total (Network.java:379-393), in place of getGradNorm(layer). */
    public float gradSumSq() {
        return OmegaHip.gradSumSq(ctx, moe);
    }

    /** tensorOP.mul(layer.diffW, clip_coef, layer.diffW) for every gradient of the layer (Network.java:401-431). */
    public void scaleGrad(float coef) {
        OmegaHip.scaleGrad(ctx, moe, coef);
    }

    /** Expert ids [T*K], combine weights [T*K], per-expert counts [E] of the last forward. */
    public void getRouting(int[] ids, float[] w, int[] counts) {
        OmegaHip.getRouting(ctx, moe, number, ids, w, counts);
    }

    // ---- checkpoint: raw little-endian float32, no header (ModelUtils.java:58-93): gate, (gate bias), then per
    // expert w1, w3, w2 - routed experts, then shared - the order LlamaMLPLayer.saveModel writes one MLP
    // (LlamaMLPLayer.java:273-283) ----

    private interface ParamVisitor {
        void visit(int which, int g, int n) throws IOException;
    }

    private void eachParam(ParamVisitor f) throws IOException {
        f.visit(OmegaHip.W_GATE, 0, nExperts * embedDim);
        if (gateBias) {
            f.visit(OmegaHip.W_GATE_BIAS, 0, nExperts);
        }
        for (int g = 0; g < nExperts + nShared; g++) {
            f.visit(OmegaHip.W_W1, g, hidden * embedDim);
            f.visit(OmegaHip.W_W3, g, hidden * embedDim);
            f.visit(OmegaHip.W_W2, g, hidden * embedDim);
        }
    }

    private static void writeFloats(RandomAccessFile out, float[] h) throws IOException {
        ByteBuffer b = ByteBuffer.allocate(4 * h.length).order(ByteOrder.LITTLE_ENDIAN);
        b.asFloatBuffer().put(h);
        out.write(b.array());
    }

    private static float[] readFloats(RandomAccessFile in, int n) throws IOException {
        byte[] raw = new byte[4 * n];
        in.readFully(raw);                         // EOFException when the checkpoint ends early
        float[] h = new float[n];
        ByteBuffer.wrap(raw).order(ByteOrder.LITTLE_ENDIAN).asFloatBuffer().get(h);
        return h;
    }

    public void saveModel(RandomAccessFile outputStream) throws IOException {
        eachParam((which, g, n) -> writeFloats(outputStream, download(which, g, n)));
    }

    public void loadModel(RandomAccessFile inputStream) throws IOException {
        eachParam((which, g, n) -> upload(which, g, readFloats(inputStream, n)));
    }

    /** The block form's parameters in the order LlamaTransformerBlock.saveModel writes its FFN half: norm2 (gamma), then
     *  the mlp (LlamaTransformerBlock.java:263-275). */
    public void saveModelBlock(RandomAccessFile outputStream) throws IOException {
        writeFloats(outputStream, download(OmegaHip.W_NORM, 0, embedDim));
        saveModel(outputStream);
    }

    public void loadModelBlock(RandomAccessFile inputStream) throws IOException {
        setNorm(readFloats(inputStream, embedDim));
        loadModel(inputStream);
    }
}

/*
 * NOT COMPILED BY THIS BUILD: neither the build image nor the GPU machines have a JDK.  This is the block a maintainer
 * adds to Omega-AI next to MoELayer (src/main/java/com/omega/engine/nn/layer/moe/LlamaMoETransformerBlock.java).
 *
 * It is LlamaTransformerBlock (J/engine/nn/layer/llama/LlamaTransformerBlock.java) with MoELayer in the FFN slot
 * (:97 setMlp(new LlamaMLPLayer(...)), :134-136 norm2 -> mlp -> add).  The attention half is the reference's own,
 * untouched, and so needs the reference's GPU backend (JCuda); the FFN half runs through libomega_hip.so.  The two
 * meet in host memory: the attention half's tensors are synchronised to the host (Tensor.syncHost, Tensor.java:559-565)
 * before MoELayer takes them, and MoELayer's results are host tensors.  End to end on one machine this therefore
 * needs either an AMD backend for the attention half or a HIP device beside the CUDA one; what the file pins down is
 * the wiring, the gradient flow and the checkpoint order.
 */
package com.omega.engine.nn.layer.moe;

import java.io.IOException;
import java.io.RandomAccessFile;

import com.omega.engine.gpu.hip.OmegaHip;
import com.omega.engine.nn.layer.Layer;
import com.omega.engine.nn.layer.LayerType;
import com.omega.engine.nn.layer.llama.LlamaAttentionLayer;
import com.omega.engine.nn.layer.llama.LlamaCausalSelfAttention2Layer;
import com.omega.engine.nn.layer.llama.LlamaFlashAttentionLayer;
import com.omega.engine.nn.layer.normalization.RMSLayer;
import com.omega.engine.nn.network.Network;
import com.omega.engine.tensor.Tensor;
import com.omega.engine.updater.UpdaterFactory;

/**
 * Transformer decoder block with a mixture-of-experts FFN:
 * <pre>
 *   tmp1   = input + attn(norm1(input))                       LlamaTransformerBlock.java:131-133
 *   output = tmp1 + moe(norm2(tmp1))                          :134-136, one native call (MoELayer.forwardBlock)
 * </pre>
 * norm2 lives inside the MoE layer: its weight is the layer's W_NORM parameter (setNorm2Weight), the normalisation,
 * the layer and the residual add are one call, and backBlock returns the gradient with respect to tmp1 with the
 * residual branch already added (:156-158).
 */
public class LlamaMoETransformerBlock extends Layer {
    private int time;
    private final int headNum, nKVHeads, embedDim;
    private final boolean bias, dropout, flashAttention;
    private LlamaAttentionLayer attn;
    private RMSLayer norm1;
    private MoELayer moe;
    private Tensor tmp1, tmp2;

    /** headNum .. network as LlamaTransformerBlock's widest constructor (:70-87); hidden .. nShared as MoELayer's. */
    public LlamaMoETransformerBlock(int headNum, int nKVHeads, int time, int embedDim, boolean bias, boolean dropout,
                                    boolean flashAttention, int hidden, int nExperts, int topK, boolean renorm, int nShared,
                                    Network network) {
        this.flashAttention = flashAttention;
        this.headNum = headNum;
        this.nKVHeads = nKVHeads;
        this.network = network;
        if (this.updater == null) {
            this.setUpdater(UpdaterFactory.create(network));
        }
        this.time = time;
        this.embedDim = embedDim;
        this.bias = bias;
        this.dropout = dropout;
        this.oChannel = 1;
        this.oHeight = 1;
        this.oWidth = embedDim;
        this.initLayers(hidden, nExperts, topK, renorm, nShared);
    }

    private void initLayers(int hidden, int nExperts, int topK, boolean renorm, int nShared) {   // :89-98
        this.norm1 = new RMSLayer(this);
        if (flashAttention) {
            this.attn = new LlamaFlashAttentionLayer(embedDim, headNum, time, bias, dropout, network);
        } else {
            this.attn = new LlamaCausalSelfAttention2Layer(embedDim, headNum, nKVHeads, time, bias, dropout, network);
        }
        this.moe = new MoELayer(embedDim, hidden, nExperts, topK, renorm, nShared, false, network);
        float[] ones = new float[embedDim];            // RMSLayer starts its weight at one (RMSLayer.initParam)
        java.util.Arrays.fill(ones, 1.0f);
        this.moe.setNorm(ones);
    }

    /** The weight of the norm in front of the FFN (norm2 of the reference block). */
    public void setNorm2Weight(float[] gamma) {
        moe.setNorm(gamma);
    }

    @Override
    public void init() {                               // :100-112
        this.number = this.input.number;
        this.time = this.network.time;
        if (this.tmp1 == null || this.tmp1.number != this.number) {
            this.tmp1 = Tensor.createGPUTensor(this.tmp1, number, 1, 1, embedDim, true);
            this.tmp2 = Tensor.createGPUTensor(this.tmp2, number, 1, 1, embedDim, true);
        }
    }

    public void output(Tensor cos, Tensor sin) {       // :129-138
        norm1.forward(input);
        attn.forward(cos, sin, norm1.getOutput());
        Tensor_OP().add(attn.getOutput(), input, tmp1);
        tmp1.syncHost();                               // the FFN half reads host tensors
        moe.forwardBlock(tmp1);                        // norm2 -> experts -> + tmp1
        this.output = moe.getOutput();
    }

    public void diff(Tensor cos, Tensor sin) {         // :150-166
        delta.syncHost();
        moe.backBlock(delta);                          // mlp.back(delta); norm2.back(mlp.diff); + delta
        Tensor gNorm2 = moe.diff;                      // gradient with respect to tmp1
        gNorm2.hostToDevice();
        attn.back(cos, sin, gNorm2);
        norm1.back(attn.diff);
        Tensor_OP().add(norm1.diff, gNorm2, tmp2);
        this.diff = tmp2;
    }

    public void forward(Tensor cos, Tensor sin, Tensor input) {   // :185-203
        this.setInput(input);
        this.init();
        this.output(cos, sin);
    }

    public void back(Tensor cos, Tensor sin, Tensor delta) {      // :210-225
        this.initBack();
        this.setDelta(delta);
        this.diff(cos, sin);
    }

    @Override
    public void update() {                             // :227-234
        norm1.update();
        attn.update();
        moe.update();                                  // gate, norm2 weight and experts, inside the native handle
    }

    @Override
    public void accGrad(float scale) {                 // :322-329
        norm1.accGrad(scale);
        attn.accGrad(scale);
        moe.accGrad(scale);
    }

    /** Checkpoint order of LlamaTransformerBlock.saveModel (:263-268): norm1, attn, norm2, mlp - the last two are the
     *  MoE layer's block form (norm weight, gate, gate bias, then W1, W3, W2 per expert). */
    public void saveModel(RandomAccessFile outputStream) throws IOException {
        norm1.saveModel(outputStream);
        attn.saveModel(outputStream);
        moe.saveModelBlock(outputStream);
    }

    public void loadModel(RandomAccessFile inputStream) throws IOException {   // :270-275
        norm1.loadModel(inputStream);
        attn.loadModel(inputStream);
        moe.loadModelBlock(inputStream);
    }

    /** The attention half registers its tensors with the network (:277-289); the MoE layer's parameters and
     *  gradients stay in the native handle - its share of a gradient norm is moe.gradSumSq(), the clipping factor is
     *  applied with moe.scaleGrad(coef) (what Network.clipGradNorm does to registered tensors, Network.java:379-432). */
    public void putParamters() {
        norm1.putParamters();
        attn.putParamters();
    }

    public void putParamterGrads() {
        norm1.putParamterGrads();
        attn.putParamterGrads();
    }

    public MoELayer getMoe() {
        return moe;
    }

    public LlamaAttentionLayer getAttn() {
        return attn;
    }

    public RMSLayer getNorm1() {
        return norm1;
    }

    @Override
    public Tensor getOutput() {
        return output;
    }

    @Override
    public LayerType getLayerType() {
        return LayerType.transformer_decoder;
    }

    // ---- the hooks the reference block leaves empty as well (:114-127, 145-148, 168-183, 205-208, 236-261) ----
    @Override
    public void initBack() {
    }

    @Override
    public void initParam() {
    }

    @Override
    public void output() {
    }

    @Override
    public void diff() {
    }

    @Override
    public void forward() {
    }

    @Override
    public void back() {
    }

    @Override
    public void forward(Tensor input) {
    }

    @Override
    public void back(Tensor delta) {
    }

    @Override
    public void showDiff() {
    }

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
}

// Drives omega::MoELayer the way a transformer block drives its FFN slot
// (J/engine/nn/layer/llama/LlamaTransformerBlock.java:135: getMlp().forward(norm2.getOutput())).
// Reads inputs and weights as raw little-endian float32 files, runs forward (and backward, block form), writes the
// outputs and the routing; used by tests/test_gpu_host_cpp.py, which compares against the CPU oracle.
//   moe_host_demo <dir> T d E K H Es renorm dtype(0|1)
#include <cstdlib>
#include <cstring>

#include "MoELayer.hpp"

static std::vector<float> read_f32(const std::string &path, size_t n)
{
    std::vector<float> v(n);
    FILE *f = fopen(path.c_str(), "rb");
    if (!f || fread(v.data(), 4, n, f) != n) throw std::runtime_error("cannot read " + path);
    fclose(f);
    return v;
}

int main(int argc, char **argv)
{
    if (argc != 10) { fprintf(stderr, "usage: %s dir T d E K H Es renorm dtype\n", argv[0]); return 2; }
    try {
        const std::string dir = argv[1];
        const int T = atoi(argv[2]), d = atoi(argv[3]), E = atoi(argv[4]), K = atoi(argv[5]), H = atoi(argv[6]),
                  Es = atoi(argv[7]), renorm = atoi(argv[8]), dtype = atoi(argv[9]);
        omega::Context ctx(0);
        omega::MoELayer mlp(d, H, E, K, renorm != 0, Es, false, ctx, dtype);
        FILE *ck = fopen((dir + "/model.bin").c_str(), "rb");
        if (!ck) throw std::runtime_error("cannot open model.bin");
        mlp.loadModel(ck);
        fclose(ck);
        omega::Tensor x(T, 1, 1, d, &ctx, true);
        x.data = read_f32(dir + "/x.bin", (size_t)T * d);
        x.hostToDevice();
        mlp.forward(x);
        omega::Tensor *out = mlp.getOutput();
        out->syncHost();
        FILE *fo = fopen((dir + "/out.bin").c_str(), "wb");
        fwrite(out->data.data(), 4, out->data.size(), fo);
        fclose(fo);
        std::vector<int32_t> ids, counts;
        std::vector<float> w;
        mlp.getRouting(ids, w, counts);
        FILE *fi = fopen((dir + "/ids.bin").c_str(), "wb");
        fwrite(ids.data(), 4, ids.size(), fi);
        fclose(fi);
        // backward, when the directory holds an output gradient: dx and two parameter gradients
        if (FILE *fd = fopen((dir + "/dout.bin").c_str(), "rb")) {
            fclose(fd);
            omega::Tensor delta(T, 1, 1, d, &ctx, true);
            delta.data = read_f32(dir + "/dout.bin", (size_t)T * d);
            delta.hostToDevice();
            mlp.back(delta);
            omega::Tensor *dx = mlp.getDiff();
            dx->syncHost();
            FILE *fx = fopen((dir + "/dx.bin").c_str(), "wb");
            fwrite(dx->data.data(), 4, dx->data.size(), fx);
            fclose(fx);
            const std::vector<float> g2 = mlp.grad(OMEGA_W_W2, E - 1), gg = mlp.grad(OMEGA_W_GATE);
            FILE *fg2 = fopen((dir + "/dW2_last.bin").c_str(), "wb");
            fwrite(g2.data(), 4, g2.size(), fg2);
            fclose(fg2);
            FILE *fgg = fopen((dir + "/dWg.bin").c_str(), "wb");
            fwrite(gg.data(), 4, gg.size(), fgg);
            fclose(fgg);
        }
        // block form (norm2 -> mlp -> residual add), when the directory holds the norm weight
        if (FILE *fg = fopen((dir + "/gamma.bin").c_str(), "rb")) {
            fclose(fg);
            std::vector<float> gamma = read_f32(dir + "/gamma.bin", (size_t)d);
            mlp.setNorm(gamma.data());
            mlp.forwardBlock(x);
            omega::Tensor *ob = mlp.getOutput();
            ob->syncHost();
            FILE *fb = fopen((dir + "/out_block.bin").c_str(), "wb");
            fwrite(ob->data.data(), 4, ob->data.size(), fb);
            fclose(fb);
            if (FILE *fd2 = fopen((dir + "/dout.bin").c_str(), "rb")) {
                fclose(fd2);
                omega::Tensor delta(T, 1, 1, d, &ctx, true);
                delta.data = read_f32(dir + "/dout.bin", (size_t)T * d);
                delta.hostToDevice();
                mlp.backBlock(delta);
                omega::Tensor *dxb = mlp.getDiff();
                dxb->syncHost();
                FILE *fxb = fopen((dir + "/dx_block.bin").c_str(), "wb");
                fwrite(dxb->data.data(), 4, dxb->data.size(), fxb);
                fclose(fxb);
                const std::vector<float> dgm = mlp.grad(OMEGA_W_NORM);
                FILE *fgm = fopen((dir + "/dgamma.bin").c_str(), "wb");
                fwrite(dgm.data(), 4, dgm.size(), fgm);
                fclose(fgm);
            }
        }
        // round trip of the checkpoint format
        FILE *sv = fopen((dir + "/model_saved.bin").c_str(), "wb");
        mlp.saveModel(sv);
        fclose(sv);
        // one optimiser step on the gradients of the last backward pass, as a Network would drive it: the layer's term
        // of the global gradient norm, the clip, AdamW at train_time 1; then the block-order checkpoint
        if (FILE *fd3 = fopen((dir + "/gamma.bin").c_str(), "rb")) {
            fclose(fd3);
            if (FILE *fd4 = fopen((dir + "/dout.bin").c_str(), "rb")) {
                fclose(fd4);
                const float ss = mlp.gradSumSq();
                FILE *fs = fopen((dir + "/gradsumsq.bin").c_str(), "wb");
                fwrite(&ss, 4, 1, fs);
                fclose(fs);
                mlp.scaleGrad(0.5f);
                const float ss2 = mlp.gradSumSq();
                if (!(ss2 > 0.24f * ss && ss2 < 0.26f * ss)) throw std::runtime_error("scaleGrad(0.5) did not quarter the sum of squares");
                mlp.updateAdamW(2e-3f, 1, 0.9f, 0.95f, 0.0f);
                FILE *st = fopen((dir + "/model_step.bin").c_str(), "wb");
                mlp.saveModelBlock(st);
                fclose(st);
            }
        }
        // error convention: a mismatching input must raise, not crash
        omega::Tensor bad(T, 1, 1, d + 1, &ctx, true);
        bool raised = false;
        try { mlp.forward(bad); } catch (const std::runtime_error &) { raised = true; }
        if (!raised) throw std::runtime_error("mismatching input was accepted");
        // a backward pass must follow a plain forward: after forwardBlock / a failed forward it raises
        omega::Tensor delta2(T, 1, 1, d + 1, &ctx, true);
        try { mlp.back(delta2); raised = false; } catch (const std::runtime_error &) { raised = true; }
        if (!raised) throw std::runtime_error("mismatching delta was accepted");
        printf("ok layerType=%s T=%d\n", mlp.getLayerType(), T);
        return 0;
    } catch (const std::exception &e) {
        fprintf(stderr, "moe_host_demo: %s\n", e.what());
        return 1;
    }
}

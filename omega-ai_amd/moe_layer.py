"""Host side of the MoE layer over the C ABI, mirroring the reference's Layer contract.

The reference is Java; no JDK is available to this build, so the host-side mirror used by the
tests and the benchmark is this module (and host/MoELayer.hpp for C++ callers).  Method names,
argument meaning and error behaviour follow the reference's layers:
  * constructor in the house style of LlamaMLPLayer(embedDim, nChannel, multiple_of, bias, network)
    (J/engine/nn/layer/llama/LlamaMLPLayer.java:47-63) with the explicit hidden size of
    DiTSwiGLUFFN (J/engine/nn/layer/dit/org/DiTSwiGLUFFN.java)
  * forward(input) = setInput -> init -> output (LlamaMLPLayer.java:200-217); getOutput()
  * saveModel/loadModel: raw little-endian float32, no header, fixed order
    (J/engine/nn/network/utils/ModelUtils.java:58-93; order w1,w3,w2 per expert as LlamaMLPLayer.java:273-283)
  * a non-zero status from the library raises RuntimeError("Error code N:msg"), the checkCUDA style
    (J/engine/gpu/CUDAMemoryManager.java:179-201)
  * back(delta) = initBack -> setDelta -> diff (LlamaMLPLayer.java:186-199), accGrad(scale) and update() without an
    updater (J/engine/nn/layer/FullyLayer.java:569-607); forward_block / back_block = the second half of
    LlamaTransformerBlock (norm2 -> mlp -> residual add and its backward, LlamaTransformerBlock.java:134-136,156-158)
"""
import ctypes as C

import numpy as np

from . import _lib as L


def _check(st, ctx_handle):
    if st != L.OK:
        msg = L.load_library().omega_hip_last_error(ctx_handle)
        raise RuntimeError((msg or b"Error code %d" % st).decode())


def f32_to_bf16_bits(a):
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    u = (u + np.uint64(0x7FFF) + ((u >> np.uint64(16)) & np.uint64(1))) >> np.uint64(16)
    return u.astype(np.uint16)


def bf16_bits_to_f32(b):
    return (np.ascontiguousarray(b, np.uint16).astype(np.uint32) << 16).view(np.float32)


class Context:
    """One device + one stream (replaces CUDAManager / CUDAPool for this path)."""

    def __init__(self, device=0):
        self.lib = L.load_library()
        h = C.c_void_p()
        st = self.lib.omega_hip_ctx_create(device, C.byref(h))
        if st != L.OK:
            raise RuntimeError((self.lib.omega_hip_last_error(None) or b"ctx_create failed").decode())
        self.handle = h

    def check(self, st):
        _check(st, self.handle)

    def sync(self):
        self.check(self.lib.omega_hip_sync(self.handle))

    def close(self):
        if self.handle:
            self.lib.omega_hip_ctx_destroy(self.handle)
            self.handle = None


class DeviceBuffer:
    """Caller-owned device memory (the role of Tensor.gpuData, J/engine/tensor/Tensor.java:23-47)."""

    def __init__(self, ctx, shape, dtype):
        self.ctx, self.shape, self.dtype = ctx, tuple(shape), dtype
        self.esize = 2 if dtype == "bf16" else 4
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.esize
        p = C.c_void_p()
        ctx.check(ctx.lib.omega_hip_malloc(ctx.handle, max(self.nbytes, 16), C.byref(p)))
        self.ptr = p

    @classmethod
    def from_numpy(cls, ctx, a, dtype):
        """a: fp32 values; stored as fp32 or as bf16 (round to nearest even)."""
        b = cls(ctx, a.shape, dtype)
        b.upload(a)
        return b

    def upload(self, a):
        h = f32_to_bf16_bits(a) if self.dtype == "bf16" else np.ascontiguousarray(a, np.float32)
        assert h.nbytes == self.nbytes
        self.ctx.check(self.ctx.lib.omega_hip_memcpy_h2d(self.ctx.handle, self.ptr, h.ctypes.data, h.nbytes))

    def to_numpy(self):
        """Blocking copy to host (Tensor.syncHost); bf16 buffers come back widened to fp32."""
        h = np.empty(self.shape, np.uint16 if self.dtype == "bf16" else np.float32)
        self.ctx.check(self.ctx.lib.omega_hip_memcpy_d2h(self.ctx.handle, h.ctypes.data, self.ptr, h.nbytes))
        return bf16_bits_to_f32(h) if self.dtype == "bf16" else h

    def fill_normal(self, seed, stream, std, first=0):
        n = int(np.prod(self.shape, dtype=np.int64))
        self.ctx.check(self.ctx.lib.omega_hip_fill_normal(self.ctx.handle, self.ptr, n, seed, stream, float(std), first,
                                                          L.DTYPE_BF16 if self.dtype == "bf16" else L.DTYPE_F32))

    def free(self):
        if self.ptr:
            self.ctx.lib.omega_hip_free(self.ctx.handle, self.ptr)
            self.ptr = None


class MoELayer:
    """Mixture-of-experts FFN layer: forward, block form, backward and the plain update."""

    def __init__(self, embedDim, hidden, nExperts, topK, renorm=True, nShared=0, bias=False, ctx=None,
                 dtype="f32", router_mode="exact", T_max=0):
        self.ctx = ctx or Context(0)
        self.lib = self.ctx.lib
        self.embedDim, self.hidden, self.nExperts, self.topK = embedDim, hidden, nExperts, topK
        self.renorm, self.nShared, self.hasBias, self.dtype = bool(renorm), nShared, bool(bias), dtype
        self.oChannel, self.oHeight, self.oWidth = 1, 1, embedDim
        self.number = 0
        self.input = None
        self.output_buf = None
        self.diff = None
        self.delta = None
        self.freeze = False
        cfg = L.MoEConfigStruct(T_max, embedDim, nExperts, topK, hidden, nShared, int(renorm), int(bias),
                                L.DTYPE_BF16 if dtype == "bf16" else L.DTYPE_F32,
                                L.ROUTER_EXACT if router_mode == "exact" else L.ROUTER_FAST)
        h = C.c_void_p()
        self.ctx.check(self.lib.omega_moe_create(self.ctx.handle, C.byref(cfg), C.byref(h)))
        self.handle = h

    # ---- parameters
    def _upload(self, which, expert, a):
        if which in (L.W_GATE_BIAS, L.W_NORM) or self.dtype == "f32":
            h = np.ascontiguousarray(a, np.float32)
        else:
            h = f32_to_bf16_bits(a)
        self.ctx.check(self.lib.omega_moe_set_weights(self.handle, which, expert, h.ctypes.data, 0))

    def set_gate(self, Wg, bg=None):
        assert Wg.shape == (self.nExperts, self.embedDim)
        self._upload(L.W_GATE, 0, Wg)
        if bg is not None:
            assert self.hasBias and bg.shape == (self.nExperts,)
            self._upload(L.W_GATE_BIAS, 0, bg)

    def set_norm(self, gamma):
        """Weight of the RMSNorm in front of the layer (block form, forward_block); always fp32."""
        assert gamma.shape == (self.embedDim,)
        self._upload(L.W_NORM, 0, gamma)

    def set_expert(self, g, W1, W3, W2):
        assert W1.shape == (self.hidden, self.embedDim) and W3.shape == W1.shape
        assert W2.shape == (self.embedDim, self.hidden)
        self._upload(L.W_W1, g, W1)
        self._upload(L.W_W3, g, W3)
        self._upload(L.W_W2, g, W2)

    def init_synthetic(self, seed, cfgmod, cfg):
        """Fills every weight on the device from the seeded generator (see configs.py): each tensor is drawn
        into a row-major scratch buffer and handed to set_weights as a device source."""
        dt = L.DTYPE_BF16 if self.dtype == "bf16" else L.DTYPE_F32
        fill = self.lib.omega_hip_fill_normal
        n_w = self.hidden * self.embedDim
        tmp = DeviceBuffer(self.ctx, (max(n_w, self.nExperts * self.embedDim),), self.dtype)
        self.ctx.check(fill(self.ctx.handle, tmp.ptr, self.nExperts * self.embedDim, seed, cfgmod.STREAM_WG,
                            cfgmod.tensor_std(cfg, "Wg"), 0, dt))
        self.ctx.check(self.lib.omega_moe_set_weights(self.handle, L.W_GATE, 0, tmp.ptr, 1))
        for g in range(self.nExperts + self.nShared):
            for which, name in ((L.W_W1, "W1"), (L.W_W3, "W3"), (L.W_W2, "W2")):
                self.ctx.check(fill(self.ctx.handle, tmp.ptr, n_w, seed, cfgmod.expert_stream(g, name),
                                    cfgmod.tensor_std(cfg, name), 0, dt))
                self.ctx.check(self.lib.omega_moe_set_weights(self.handle, which, g, tmp.ptr, 1))
        tmp.free()
        bg = cfgmod.zipf_gate_bias(cfg, seed)
        if bg is not None:
            self._upload(L.W_GATE_BIAS, 0, bg)
        # norm weight of the block form: 1 + 0.1 * N(0,1), drawn on the device as fp32
        gam = DeviceBuffer(self.ctx, (self.embedDim,), "f32")
        self.ctx.check(fill(self.ctx.handle, gam.ptr, self.embedDim, seed, cfgmod.STREAM_NORM, 1.0, 0, L.DTYPE_F32))
        g = gam.to_numpy() * np.float32(0.1) + np.float32(1.0)
        gam.free()
        self.set_norm(g.astype(np.float32))
        self.ctx.sync()

    # ---- Layer contract
    def init(self):
        """(Re)allocates the output when the batch size changes (LlamaMLPLayer.init)."""
        self.number = self.input.shape[0]
        if self.output_buf is None or self.output_buf.shape[0] != self.number:
            if self.output_buf is not None:
                self.output_buf.free()
            self.output_buf = DeviceBuffer(self.ctx, (self.number, self.embedDim), self.dtype)

    def setInput(self, inp):
        if inp.shape[-1] != self.embedDim:
            raise RuntimeError("Error code 1:input width does not match embedDim")
        self.input = inp

    def output(self):
        self.ctx.check(self.lib.omega_moe_forward(self.handle, self.input.ptr, self.number, self.output_buf.ptr))

    def forward(self, inp):
        self.setInput(inp)
        self.init()
        self.output()
        return self.output_buf

    def forward_block(self, inp):
        """out = inp + layer(rmsnorm(inp)): norm2 -> mlp -> residual add of LlamaTransformerBlock.output
        (J/engine/nn/layer/llama/LlamaTransformerBlock.java:134-136) in one call."""
        self.setInput(inp)
        self.init()
        self.ctx.check(self.lib.omega_moe_forward_block(self.handle, self.input.ptr, self.number, self.output_buf.ptr))
        return self.output_buf

    def norm_rms(self, T=None):
        """rms[t] of the last forward_block (host copy)."""
        T = self.number if T is None else T
        r = np.empty(T, np.float32)
        self.ctx.check(self.lib.omega_moe_get_norm(self.handle, T, r.ctypes.data))
        return r

    def getOutput(self):
        return self.output_buf

    def getLayerType(self):
        return "feed_forward"

    # the hooks LlamaMLPLayer leaves empty (J/engine/nn/layer/llama/LlamaMLPLayer.java:247-271)
    def backTemp(self):
        pass

    def showDiff(self):
        pass

    def initCache(self):
        pass

    def set_training(self, on=True):
        """Forward keeps h1 / h3 for back(), as the reference's layers keep their outputs."""
        self.ctx.check(self.lib.omega_moe_set_training(self.handle, int(bool(on))))

    def set_gather_mode(self, mode):
        """How the rows of x reach the experts of a bf16 layer: 0 by shape, 1 gathered copy, 2 fetched by the up
        product's loads (omega_moe_set_gather_mode)."""
        self.ctx.check(self.lib.omega_moe_set_gather_mode(self.handle, int(mode)))

    def gather_on_load(self):
        """True if the last dispatch left the rows of x to the up product's loads (no gathered copy)."""
        return bool(self.lib.omega_moe_gather_on_load(self.handle))

    def initBack(self):
        """(Re)allocates the input gradient when the batch size changes (FullyLayer.initBack,
        J/engine/nn/layer/FullyLayer.java:130-144); the parameter gradients live in the native handle."""
        if self.diff is None or self.diff.shape[0] != self.number:
            if self.diff is not None:
                self.diff.free()
            self.diff = DeviceBuffer(self.ctx, (self.number, self.embedDim), self.dtype)

    def back(self, delta):
        """back(Tensor delta) = initBack -> setDelta -> diff (LlamaMLPLayer.back,
        J/engine/nn/layer/llama/LlamaMLPLayer.java:186-199): input gradient returned, parameter gradients overwritten.
        Must follow forward() of the same input."""
        if self.input is None:
            raise RuntimeError("Error code 1:back without a forward")
        if tuple(delta.shape) != (self.number, self.embedDim):
            raise RuntimeError("Error code 1:delta shape does not match the output")
        self.initBack()
        self.delta = delta
        self.ctx.check(self.lib.omega_moe_backward(self.handle, self.input.ptr, delta.ptr, self.number, self.diff.ptr))
        return self.diff

    def back_block(self, delta):
        """Backward of forward_block: mlp.back(delta); norm2.back(mlp.diff); add(norm2.diff, delta)
        (J/engine/nn/layer/llama/LlamaTransformerBlock.java:156-158).  Returns the gradient of the block's input; the
        gradient of the norm weight is grad(W_NORM)."""
        if self.input is None:
            raise RuntimeError("Error code 1:back without a forward")
        if tuple(delta.shape) != (self.number, self.embedDim):
            raise RuntimeError("Error code 1:delta shape does not match the output")
        self.initBack()
        self.delta = delta
        self.ctx.check(self.lib.omega_moe_backward_block(self.handle, self.input.ptr, delta.ptr, self.number, self.diff.ptr))
        return self.diff

    def grad(self, which, expert=0):
        """Host copy of one parameter gradient (fp32), in the layout of its weight."""
        shape = {L.W_GATE: (self.nExperts, self.embedDim), L.W_GATE_BIAS: (self.nExperts,), L.W_NORM: (self.embedDim,),
                 L.W_W1: (self.hidden, self.embedDim), L.W_W3: (self.hidden, self.embedDim),
                 L.W_W2: (self.embedDim, self.hidden)}[which]
        g = np.empty(shape, np.float32)
        self.ctx.check(self.lib.omega_moe_get_grad(self.handle, which, expert, g.ctypes.data, 0))
        return g

    def accGrad(self, scale):
        self.ctx.check(self.lib.omega_moe_acc_grad(self.handle, float(scale)))

    def gradSumSq(self):
        """Sum of the squares of every parameter gradient of the layer (of the accumulators once accGrad has run): the
        layer's term of Network.clipGradNorm's total (J/engine/nn/network/Network.java:379-393)."""
        v = C.c_float(0.0)
        self.ctx.check(self.lib.omega_moe_grad_sumsq(self.handle, C.byref(v)))
        return float(v.value)

    def scaleGrad(self, coef):
        """Gradients (or accumulators) times coef (tensorOP.mul(diffW, clip_coef, diffW), Network.java:401-431)."""
        self.ctx.check(self.lib.omega_moe_scale_grad(self.handle, float(coef)))

    def clipGradNorm(self, gradClip, other_sumsq=0.0):
        """Network.clipGradNorm (Network.java:379-432) for a network whose other layers contribute other_sumsq:
        clip_coef = min(1, gradClip / (sqrt(total) + 1e-6)) in float as there, applied to this layer.  Returns it."""
        total = np.float32(np.float32(other_sumsq) + np.float32(self.gradSumSq()))
        coef = np.float32(gradClip / (np.sqrt(np.float64(total)) + np.float64(np.float32(1e-6))))
        if coef > 1:
            coef = np.float32(1.0)
        self.scaleGrad(coef)
        return float(coef)

    def update(self, learnRate):
        """The update of a layer without an updater: w -= learnRate * diffW (FullyLayer.update,
        J/engine/nn/layer/FullyLayer.java:569-590); bf16 layers step fp32 master copies and re-round.  forward() must run
        again before the next back()."""
        if self.freeze:      # Layer.freeze: a frozen layer's update() does nothing (FullyLayer.java:571)
            return
        self.ctx.check(self.lib.omega_moe_update(self.handle, float(learnRate)))

    def updateAdamW(self, learnRate, train_time, beta1=0.9, beta2=0.95, weight_decay=1e-4):
        """update() under the AdamW updater (AdamW.update, J/engine/updater/AdamW.java:69-92; adamw_kernel,
        J/engine/updater/gpu/updater.cu:31-52): train_time is network.train_time, starting at 1; the defaults are the
        reference's (AdamWKernel.java:25-26, AdamW.java:27).  forward() must run again before the next back()."""
        if self.freeze:
            return
        self.ctx.check(self.lib.omega_moe_update_adamw(self.handle, float(learnRate), float(beta1), float(beta2),
                                                       float(weight_decay), int(train_time)))

    # ---- stages and introspection
    def stage(self, name, x=None, out=None):
        T = self.number
        f = {"router": lambda: self.lib.omega_moe_router(self.handle, x.ptr, T),
             "dispatch": lambda: self.lib.omega_moe_dispatch(self.handle, x.ptr, T),
             "experts": lambda: self.lib.omega_moe_experts(self.handle, x.ptr if x is not None else None, T),
             "combine": lambda: self.lib.omega_moe_combine(self.handle, T, out.ptr)}[name]
        self.ctx.check(f())

    def time_stage(self, stage, x, T, out=None, warmup=2, iters=10):
        ms = C.c_float()
        self.ctx.check(self.lib.omega_moe_time_stage(self.handle, stage, x.ptr if x is not None else None, T,
                                                     out.ptr if out is not None else None, warmup, iters, C.byref(ms)))
        return ms.value

    def time_backward(self, x, dout, T, dx, warmup=2, iters=10):
        ms = C.c_float()
        self.ctx.check(self.lib.omega_moe_time_backward(self.handle, x.ptr, dout.ptr, T, dx.ptr, warmup, iters, C.byref(ms)))
        return ms.value

    def set_profiling(self, on):
        self.ctx.check(self.lib.omega_moe_set_profiling(self.handle, int(on)))

    def get_profile(self):
        """(per-stage average ms dict, number of forwards) since profiling was switched on."""
        ms = (C.c_float * 5)()
        n = C.c_int()
        self.ctx.check(self.lib.omega_moe_get_profile(self.handle, ms, C.byref(n)))
        names = ("router", "dispatch", "experts_up", "experts_down", "combine")
        return {k: ms[i] / max(n.value, 1) for i, k in enumerate(names)}, n.value

    def routing(self, T=None):
        T = self.number if T is None else T
        K, E = self.topK, self.nExperts
        r = dict(ids=np.empty((T, K), np.int32), w=np.empty((T, K), np.float32), counts=np.empty(E, np.int32),
                 offsets=np.empty(E + 1, np.int32), dst=np.empty(T * K, np.int32), src_row=np.empty(T * K, np.int32))
        self.ctx.check(self.lib.omega_moe_get_routing(self.handle, T, *[r[k].ctypes.data for k in
                                                                         ("ids", "w", "counts", "offsets", "dst", "src_row")]))
        return r

    def router_probs(self, x, T):
        lg = np.empty((T, self.nExperts), np.float32)
        p = np.empty((T, self.nExperts), np.float32)
        self.ctx.check(self.lib.omega_moe_get_router_probs(self.handle, x.ptr, T, lg.ctypes.data, p.ctypes.data))
        return lg, p

    def router_probs_noalloc(self, x, T):
        """router_probs through the entry point that allocates nothing (T within T_max, T*E within 2^20)."""
        lg = np.empty((T, self.nExperts), np.float32)
        p = np.empty((T, self.nExperts), np.float32)
        self.ctx.check(self.lib.omega_moe_get_router_probs_noalloc(self.handle, x.ptr, T, lg.ctypes.data, p.ctypes.data))
        return lg, p

    def workspace(self, which, T):
        """Host copy of a workspace buffer in logical row order: 'xg' [T*K,d], 'a' [T*K+Es*T,H],
        'y' [T*K+Es*T,d] (fp32 values); after back() also 'dh' [T*K+Es*T,2H] (dh1 | dh3, bf16 layers) and
        'dlogits' [T,E]."""
        idx = {"xg": 0, "a": 1, "y": 2, "dh": 3, "dlogits": 4}[which]
        P, R = T * self.topK, T * self.topK + self.nShared * T
        shape = {"xg": (P, self.embedDim), "a": (R, self.hidden), "y": (R, self.embedDim),
                 "dh": (R, 2 * self.hidden), "dlogits": (T, self.nExperts)}[which]
        raw_bf16 = self.dtype == "bf16" and which not in ("y", "dlogits")
        h = np.zeros(shape, np.uint16 if raw_bf16 else np.float32)
        self.ctx.check(self.lib.omega_moe_get_workspace(self.handle, idx, T, h.ctypes.data))
        return bf16_bits_to_f32(h) if raw_bf16 else h

    def fill_workspace(self, which, byte_value):
        """Every byte of the 'a' or 'y' buffer (padding rows included) set to byte_value; 0xFF reads as NaN."""
        self.ctx.check(self.lib.omega_moe_fill_workspace(self.handle, {"a": 1, "y": 2}[which], int(byte_value)))

    # ---- checkpoint: raw LE float32, order gate, (gate bias), then w1,w3,w2 per expert, routed then shared
    def _download_weight(self, which, expert, shape):
        raw_bf16 = self.dtype == "bf16" and which not in (L.W_GATE_BIAS, L.W_NORM)   # those two are fp32 in every layer
        h = np.empty(shape, np.uint16 if raw_bf16 else np.float32)
        self.ctx.check(self.lib.omega_moe_get_weights(self.handle, which, expert, h.ctypes.data, 0))
        return bf16_bits_to_f32(h) if raw_bf16 else h

    def _param_list(self):
        items = [(L.W_GATE, 0, (self.nExperts, self.embedDim))]
        if self.hasBias:
            items.append((L.W_GATE_BIAS, 0, (self.nExperts,)))
        for g in range(self.nExperts + self.nShared):
            items += [(L.W_W1, g, (self.hidden, self.embedDim)), (L.W_W3, g, (self.hidden, self.embedDim)),
                      (L.W_W2, g, (self.embedDim, self.hidden))]
        return items

    def saveModel(self, f):
        for which, g, shape in self._param_list():
            f.write(self._download_weight(which, g, shape).astype("<f4").tobytes())

    def loadModel(self, f):
        for which, g, shape in self._param_list():
            n = int(np.prod(shape))
            buf = f.read(4 * n)
            if len(buf) != 4 * n:
                raise RuntimeError("Error code 1:checkpoint ends early")
            self._upload(which, g, np.frombuffer(buf, "<f4").reshape(shape))

    def saveModelBlock(self, f):
        """The block form's parameters in the order LlamaTransformerBlock.saveModel writes its FFN half: norm2 (gamma,
        RMSLayer.saveModel), then the mlp (J/engine/nn/layer/llama/LlamaTransformerBlock.java:263-275)."""
        f.write(self._download_weight(L.W_NORM, 0, (self.embedDim,)).astype("<f4").tobytes())
        self.saveModel(f)

    def loadModelBlock(self, f):
        buf = f.read(4 * self.embedDim)
        if len(buf) != 4 * self.embedDim:
            raise RuntimeError("Error code 1:checkpoint ends early")
        self.set_norm(np.frombuffer(buf, "<f4").copy())
        self.loadModel(f)

    def initJava(self, seed, mean=0.01, std=0.02):
        """RandomUtils.setSeed(seed) followed by the house-style initialisation (java_random.init_layer): the weights a
        Java run of the reference would draw.  Returns the arrays that were set."""
        from . import java_random
        return java_random.init_layer(self, java_random.JavaRandom(seed), mean, std)

    def loadJson(self, weight_map, layer_index=0, scheme="omega", strict=True):
        """Weights by name from a JSON export of a PyTorch state dict (see weights_json.py; the reference's
        LagJsonReader + ModeLoaderlUtils.loadData route)."""
        from . import weights_json
        return weights_json.load_moe_weights(self, weight_map, layer_index, scheme, strict)

    def close(self):
        if self.output_buf is not None:
            self.output_buf.free()
            self.output_buf = None
        if self.diff is not None:
            self.diff.free()
            self.diff = None
        if self.handle:
            self.lib.omega_moe_destroy(self.handle)
            self.handle = None

/*
 * NOT COMPILED BY THIS BUILD: neither the build image nor the GPU machines have a JDK.  This is the binding a
 * maintainer adds to Omega-AI (src/main/java/com/omega/engine/gpu/hip/OmegaHip.java, JDK >= 22); every call and its
 * order mirror the compiled and GPU-tested C++ twin, omega-ai_amd/host/MoELayer.hpp.
 */
package com.omega.engine.gpu.hip;

import static java.lang.foreign.ValueLayout.ADDRESS;
import static java.lang.foreign.ValueLayout.JAVA_FLOAT;
import static java.lang.foreign.ValueLayout.JAVA_INT;
import static java.lang.foreign.ValueLayout.JAVA_LONG;

import java.lang.foreign.Arena;
import java.lang.foreign.FunctionDescriptor;
import java.lang.foreign.Linker;
import java.lang.foreign.MemoryLayout;
import java.lang.foreign.MemorySegment;
import java.lang.foreign.SymbolLookup;
import java.lang.invoke.MethodHandle;

/**
 * FFM (java.lang.foreign) downcalls into libomega_hip.so, the C ABI of include/omega_hip.h.  Stands in, for the MoE
 * layer only, for CUDAManager / CUDAModules module loading (CUDAManager.java:125-159), CUDAMemoryManager
 * (CUDAMemoryManager.java:115-123) and the cuBLAS wrapper (GPUOP.java:405-417).  A non-zero status becomes
 * RuntimeException("Error code N:msg"), the style of CUDAMemoryManager.checkCUDA (CUDAMemoryManager.java:179-201).
 */
public final class OmegaHip {
    private static final Linker LINKER = Linker.nativeLinker();
    private static final SymbolLookup LIB =
            SymbolLookup.libraryLookup(System.getProperty("omega.hip.lib", "libomega_hip.so"), Arena.global());

    private static MethodHandle h(String name, FunctionDescriptor fd) {
        return LINKER.downcallHandle(LIB.find(name).orElseThrow(() -> new UnsatisfiedLinkError(name)), fd);
    }

    private static final MethodHandle CTX_CREATE = h("omega_hip_ctx_create", FunctionDescriptor.of(JAVA_INT, JAVA_INT, ADDRESS));
    private static final MethodHandle CTX_DESTROY = h("omega_hip_ctx_destroy", FunctionDescriptor.of(JAVA_INT, ADDRESS));
    private static final MethodHandle LAST_ERROR = h("omega_hip_last_error", FunctionDescriptor.of(ADDRESS, ADDRESS));
    private static final MethodHandle MALLOC = h("omega_hip_malloc", FunctionDescriptor.of(JAVA_INT, ADDRESS, JAVA_LONG, ADDRESS));
    private static final MethodHandle FREE = h("omega_hip_free", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS));
    private static final MethodHandle H2D = h("omega_hip_memcpy_h2d", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, ADDRESS, JAVA_LONG));
    private static final MethodHandle D2H = h("omega_hip_memcpy_d2h", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, ADDRESS, JAVA_LONG));
    private static final MethodHandle SYNC = h("omega_hip_sync", FunctionDescriptor.of(JAVA_INT, ADDRESS));
    private static final MethodHandle CONVERT = h("omega_hip_convert", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, JAVA_INT, ADDRESS, JAVA_INT, JAVA_LONG));
    private static final MethodHandle MOE_CREATE = h("omega_moe_create", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, ADDRESS));
    private static final MethodHandle MOE_DESTROY = h("omega_moe_destroy", FunctionDescriptor.of(JAVA_INT, ADDRESS));
    private static final MethodHandle SET_WEIGHTS = h("omega_moe_set_weights", FunctionDescriptor.of(JAVA_INT, ADDRESS, JAVA_INT, JAVA_INT, ADDRESS, JAVA_INT));
    private static final MethodHandle GET_WEIGHTS = h("omega_moe_get_weights", FunctionDescriptor.of(JAVA_INT, ADDRESS, JAVA_INT, JAVA_INT, ADDRESS, JAVA_INT));
    private static final MethodHandle FORWARD = h("omega_moe_forward", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, JAVA_INT, ADDRESS));
    private static final MethodHandle FORWARD_BLOCK = h("omega_moe_forward_block", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, JAVA_INT, ADDRESS));
    private static final MethodHandle BACKWARD = h("omega_moe_backward", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, ADDRESS, JAVA_INT, ADDRESS));
    private static final MethodHandle BACKWARD_BLOCK = h("omega_moe_backward_block", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS, ADDRESS, JAVA_INT, ADDRESS));
    private static final MethodHandle SET_TRAINING = h("omega_moe_set_training", FunctionDescriptor.of(JAVA_INT, ADDRESS, JAVA_INT));
    private static final MethodHandle SET_GATHER_MODE = h("omega_moe_set_gather_mode", FunctionDescriptor.of(JAVA_INT, ADDRESS, JAVA_INT));
    private static final MethodHandle GATHER_ON_LOAD = h("omega_moe_gather_on_load", FunctionDescriptor.of(JAVA_INT, ADDRESS));
    private static final MethodHandle GET_GRAD = h("omega_moe_get_grad", FunctionDescriptor.of(JAVA_INT, ADDRESS, JAVA_INT, JAVA_INT, ADDRESS, JAVA_INT));
    private static final MethodHandle ACC_GRAD = h("omega_moe_acc_grad", FunctionDescriptor.of(JAVA_INT, ADDRESS, JAVA_FLOAT));
    private static final MethodHandle UPDATE = h("omega_moe_update", FunctionDescriptor.of(JAVA_INT, ADDRESS, JAVA_FLOAT));
    private static final MethodHandle UPDATE_ADAMW = h("omega_moe_update_adamw", FunctionDescriptor.of(JAVA_INT, ADDRESS, JAVA_FLOAT, JAVA_FLOAT, JAVA_FLOAT, JAVA_FLOAT, JAVA_INT));
    private static final MethodHandle GRAD_SUMSQ = h("omega_moe_grad_sumsq", FunctionDescriptor.of(JAVA_INT, ADDRESS, ADDRESS));
    private static final MethodHandle SCALE_GRAD = h("omega_moe_scale_grad", FunctionDescriptor.of(JAVA_INT, ADDRESS, JAVA_FLOAT));
    private static final MethodHandle GET_ROUTING = h("omega_moe_get_routing", FunctionDescriptor.of(JAVA_INT, ADDRESS, JAVA_INT, ADDRESS, ADDRESS, ADDRESS, ADDRESS, ADDRESS, ADDRESS));

    /** struct omega_moe_config: ten int32 in declaration order. */
    private static final MemoryLayout MOE_CONFIG = MemoryLayout.structLayout(
            JAVA_INT.withName("T_max"), JAVA_INT.withName("d"), JAVA_INT.withName("E"), JAVA_INT.withName("K"),
            JAVA_INT.withName("H"), JAVA_INT.withName("Es"), JAVA_INT.withName("renorm"), JAVA_INT.withName("has_gate_bias"),
            JAVA_INT.withName("dtype"), JAVA_INT.withName("router_mode"));

    public static final int F32 = 0, BF16 = 1;
    public static final int ROUTER_EXACT = 0, ROUTER_FAST = 1;
    public static final int W_GATE = 0, W_GATE_BIAS = 1, W_W1 = 2, W_W3 = 3, W_W2 = 4, W_NORM = 5;

    private OmegaHip() {
    }

    /** Turns a non-zero status into the RuntimeException the reference's checkCUDA throws. */
    static void check(MemorySegment ctx, int status) {
        if (status == 0) {
            return;
        }
        String msg = "Error code " + status;
        try {
            MemorySegment p = (MemorySegment) LAST_ERROR.invokeExact(ctx);
            if (!p.equals(MemorySegment.NULL)) {
                String s = p.reinterpret(1024).getString(0);
                if (!s.isEmpty()) {
                    msg = s;
                }
            }
        } catch (Throwable t) {
            // keep the bare status
        }
        throw new RuntimeException(msg);
    }

    private static RuntimeException wrap(Throwable t) {
        return t instanceof RuntimeException r ? r : new RuntimeException(t);
    }

    // ---- context and device memory (device addresses travel as long, like SerializablePointer(long)) ----

    public static MemorySegment ctxCreate(int device) {
        try (Arena a = Arena.ofConfined()) {
            MemorySegment out = a.allocate(ADDRESS);
            check(MemorySegment.NULL, (int) CTX_CREATE.invokeExact(device, out));
            return out.get(ADDRESS, 0);
        } catch (Throwable t) {
            throw wrap(t);
        }
    }

    public static void ctxDestroy(MemorySegment ctx) {
        try {
            int st = (int) CTX_DESTROY.invokeExact(ctx);
        } catch (Throwable t) {
            throw wrap(t);
        }
    }

    public static long malloc(MemorySegment ctx, long bytes) {
        try (Arena a = Arena.ofConfined()) {
            MemorySegment out = a.allocate(ADDRESS);
            check(ctx, (int) MALLOC.invokeExact(ctx, bytes, out));
            return out.get(ADDRESS, 0).address();
        } catch (Throwable t) {
            throw wrap(t);
        }
    }

    public static void free(MemorySegment ctx, long dptr) {
        if (dptr == 0L) {
            return;
        }
        try {
            check(ctx, (int) FREE.invokeExact(ctx, MemorySegment.ofAddress(dptr)));
        } catch (Throwable t) {
            throw wrap(t);
        }
    }

    /** Tensor.hostToDevice for a float[] (blocking). */
    public static void h2d(MemorySegment ctx, long dst, float[] src, int n) {
        try (Arena a = Arena.ofConfined()) {
            MemorySegment host = a.allocate(JAVA_FLOAT, n);
            MemorySegment.copy(src, 0, host, JAVA_FLOAT, 0, n);
            check(ctx, (int) H2D.invokeExact(ctx, MemorySegment.ofAddress(dst), host, 4L * n));
        } catch (Throwable t) {
            throw wrap(t);
        }
    }

    /** Tensor.syncHost into a float[] (blocking). */
    public static void d2h(MemorySegment ctx, float[] dst, long src, int n) {
        try (Arena a = Arena.ofConfined()) {
            MemorySegment host = a.allocate(JAVA_FLOAT, n);
            check(ctx, (int) D2H.invokeExact(ctx, host, MemorySegment.ofAddress(src), 4L * n));
            MemorySegment.copy(host, JAVA_FLOAT, 0, dst, 0, n);
        } catch (Throwable t) {
            throw wrap(t);
        }
    }

    public static void sync(MemorySegment ctx) {
        try {
            check(ctx, (int) SYNC.invokeExact(ctx));
        } catch (Throwable t) {
            throw wrap(t);
        }
    }

    /** fp32 <-> bf16 conversion of device buffers (n elements). */
    public static void convert(MemorySegment ctx, long dst, int dstDtype, long src, int srcDtype, long n) {
        try {
            check(ctx, (int) CONVERT.invokeExact(ctx, MemorySegment.ofAddress(dst), dstDtype, MemorySegment.ofAddress(src), srcDtype, n));
        } catch (Throwable t) {
            throw wrap(t);
        }
    }

    // ---- the layer ----

    public static MemorySegment moeCreate(MemorySegment ctx, int tMax, int d, int e, int k, int h, int es, boolean renorm,
                                          boolean gateBias, int dtype, int routerMode) {
        try (Arena a = Arena.ofConfined()) {
            MemorySegment cfg = a.allocate(MOE_CONFIG);
            int[] v = {tMax, d, e, k, h, es, renorm ? 1 : 0, gateBias ? 1 : 0, dtype, routerMode};
            for (int i = 0; i < v.length; i++) {
                cfg.setAtIndex(JAVA_INT, i, v[i]);
            }
            MemorySegment out = a.allocate(ADDRESS);
            check(ctx, (int) MOE_CREATE.invokeExact(ctx, cfg, out));
            return out.get(ADDRESS, 0);
        } catch (Throwable t) {
            throw wrap(t);
        }
    }

    public static void moeDestroy(MemorySegment moe) {
        try {
            int st = (int) MOE_DESTROY.invokeExact(moe);
        } catch (Throwable t) {
            throw wrap(t);
        }
    }

    /** One weight tensor from a device buffer holding elements of the layer dtype ([out,in] row-major). */
    public static void setWeightsDevice(MemorySegment ctx, MemorySegment moe, int which, int expert, long src) {
        try {
            check(ctx, (int) SET_WEIGHTS.invokeExact(moe, which, expert, MemorySegment.ofAddress(src), 1));
        } catch (Throwable t) {
            throw wrap(t);
        }
    }

    /** One fp32 tensor (gate bias, norm weight, or any weight of an fp32 layer) from host memory. */
    public static void setWeightsHost(MemorySegment ctx, MemorySegment moe, int which, int expert, float[] src) {
        try (Arena a = Arena.ofConfined()) {
            MemorySegment host = a.allocate(JAVA_FLOAT, src.length);
            MemorySegment.copy(src, 0, host, JAVA_FLOAT, 0, src.length);
            check(ctx, (int) SET_WEIGHTS.invokeExact(moe, which, expert, host, 0));
        } catch (Throwable t) {
            throw wrap(t);
        }
    }

    public static void getWeightsDevice(MemorySegment ctx, MemorySegment moe, int which, int expert, long dst) {
        try {
            check(ctx, (int) GET_WEIGHTS.invokeExact(moe, which, expert, MemorySegment.ofAddress(dst), 1));
        } catch (Throwable t) {
            throw wrap(t);
        }
    }

    public static void getWeightsHost(MemorySegment ctx, MemorySegment moe, int which, int expert, float[] dst) {
        try (Arena a = Arena.ofConfined()) {
            MemorySegment host = a.allocate(JAVA_FLOAT, dst.length);
            check(ctx, (int) GET_WEIGHTS.invokeExact(moe, which, expert, host, 0));
            MemorySegment.copy(host, JAVA_FLOAT, 0, dst, 0, dst.length);
        } catch (Throwable t) {
            throw wrap(t);
        }
    }

    public static void forward(MemorySegment ctx, MemorySegment moe, long x, int t, long out, boolean block) {
        try {
            MethodHandle f = block ? FORWARD_BLOCK : FORWARD;
            check(ctx, (int) f.invokeExact(moe, MemorySegment.ofAddress(x), t, MemorySegment.ofAddress(out)));
        } catch (Throwable t2) {
            throw wrap(t2);
        }
    }

    public static void backward(MemorySegment ctx, MemorySegment moe, long x, long dout, int t, long dx, boolean block) {
        try {
            MethodHandle f = block ? BACKWARD_BLOCK : BACKWARD;
            check(ctx, (int) f.invokeExact(moe, MemorySegment.ofAddress(x), MemorySegment.ofAddress(dout), t, MemorySegment.ofAddress(dx)));
        } catch (Throwable t2) {
            throw wrap(t2);
        }
    }

    public static void setTraining(MemorySegment ctx, MemorySegment moe, boolean on) {
        try {
            check(ctx, (int) SET_TRAINING.invokeExact(moe, on ? 1 : 0));
        } catch (Throwable t) {
            throw wrap(t);
        }
    }

    /** Whether the last dispatch left the rows of x to the up product's loads (omega_moe_gather_on_load). */
    public static boolean gatherOnLoad(MemorySegment moe) {
        try {
            return (int) GATHER_ON_LOAD.invokeExact(moe) != 0;
        } catch (Throwable t) {
            throw wrap(t);
        }
    }

    /** 0 by shape, 1 gathered copy, 2 rows fetched by the up product's loads (omega_moe_set_gather_mode). */
    public static void setGatherMode(MemorySegment ctx, MemorySegment moe, int mode) {
        try {
            check(ctx, (int) SET_GATHER_MODE.invokeExact(moe, mode));
        } catch (Throwable t) {
            throw wrap(t);
        }
    }

    /** One parameter gradient (always fp32, layout of its weight) into a float[]. */
    public static void getGradHost(MemorySegment ctx, MemorySegment moe, int which, int expert, float[] dst) {
        try (Arena a = Arena.ofConfined()) {
            MemorySegment host = a.allocate(JAVA_FLOAT, dst.length);
            check(ctx, (int) GET_GRAD.invokeExact(moe, which, expert, host, 0));
            MemorySegment.copy(host, JAVA_FLOAT, 0, dst, 0, dst.length);
        } catch (Throwable t) {
            throw wrap(t);
        }
    }

    public static void accGrad(MemorySegment ctx, MemorySegment moe, float scale) {
        try {
            check(ctx, (int) ACC_GRAD.invokeExact(moe, scale));
        } catch (Throwable t) {
            throw wrap(t);
        }
    }

    public static void update(MemorySegment ctx, MemorySegment moe, float lr) {
        try {
            check(ctx, (int) UPDATE.invokeExact(moe, lr));
        } catch (Throwable t) {
            throw wrap(t);
        }
    }

    public static void updateAdamW(MemorySegment ctx, MemorySegment moe, float lr, float beta1, float beta2, float weightDecay, int trainTime) {
        try {
            check(ctx, (int) UPDATE_ADAMW.invokeExact(moe, lr, beta1, beta2, weightDecay, trainTime));
        } catch (Throwable t) {
            throw wrap(t);
        }
    }

    public static float gradSumSq(MemorySegment ctx, MemorySegment moe) {
        try (Arena a = Arena.ofConfined()) {
            MemorySegment out = a.allocate(JAVA_FLOAT);
            check(ctx, (int) GRAD_SUMSQ.invokeExact(moe, out));
            return out.get(JAVA_FLOAT, 0);
        } catch (Throwable t) {
            throw wrap(t);
        }
    }

    public static void scaleGrad(MemorySegment ctx, MemorySegment moe, float coef) {
        try {
            check(ctx, (int) SCALE_GRAD.invokeExact(moe, coef));
        } catch (Throwable t) {
            throw wrap(t);
        }
    }

    /** Expert ids [T*K], combine weights [T*K] and per-expert counts [E] of the last forward (any array may be null). */
    public static void getRouting(MemorySegment ctx, MemorySegment moe, int t, int[] ids, float[] w, int[] counts) {
        try (Arena a = Arena.ofConfined()) {
            MemorySegment pi = ids == null ? MemorySegment.NULL : a.allocate(JAVA_INT, ids.length);
            MemorySegment pw = w == null ? MemorySegment.NULL : a.allocate(JAVA_FLOAT, w.length);
            MemorySegment pc = counts == null ? MemorySegment.NULL : a.allocate(JAVA_INT, counts.length);
            check(ctx, (int) GET_ROUTING.invokeExact(moe, t, pi, pw, pc, MemorySegment.NULL, MemorySegment.NULL, MemorySegment.NULL));
            if (ids != null) {
                MemorySegment.copy(pi, JAVA_INT, 0, ids, 0, ids.length);
            }
            if (w != null) {
                MemorySegment.copy(pw, JAVA_FLOAT, 0, w, 0, w.length);
            }
            if (counts != null) {
                MemorySegment.copy(pc, JAVA_INT, 0, counts, 0, counts.length);
            }
        } catch (Throwable t2) {
            throw wrap(t2);
        }
    }
}

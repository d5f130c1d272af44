"""JSON weight import for the MoE layer, in the style the reference loads exported PyTorch weights.

The reference reads a JSON object {parameter name: nested lists of numbers} into a map
(LagJsonReader.readJsonFileSmallWeight / readJsonFileBigWeightIterator,
J/example/transformer/utils/LagJsonReader.java:56-88) and copies each entry into a layer tensor by name
(ModeLoaderlUtils.loadData, J/example/common/ModeLoaderlUtils.java:1463-1508: 1-D -> data[n], 2-D row-major
-> data[n*W + w], values narrowed to float; a missing key is reported and skipped).  For the dense FFN the names
are "layers.<i>.feed_forward.w1|w2|w3.weight" and "layers.<i>.ffn_norm.weight"
(J/example/transformer/test/Llama3Test.java:677-681), with w1/w3 of shape [hidden, dim], w2 [dim, hidden]: the
[out, in] layout of FullyLayer (J/engine/nn/layer/FullyLayer.java:181) and of this layer's set_expert.

Name schemes understood (layer index i, expert e):
  "omega"     layers.<i>.feed_forward.gate.weight [E,d], layers.<i>.feed_forward.experts.<e>.w1|w3|w2.weight,
              shared experts layers.<i>.feed_forward.shared_experts.<s>.w1|w3|w2.weight,
              layers.<i>.ffn_norm.weight; with E == 1 and no experts.* keys, the dense names
              layers.<i>.feed_forward.w1|w3|w2.weight of Llama3Test are accepted for expert 0
  "mixtral"   model.layers.<i>.block_sparse_moe.gate.weight, ....experts.<e>.w1|w3|w2.weight,
              model.layers.<i>.post_attention_layernorm.weight
  "deepseek"  model.layers.<i>.mlp.gate.weight (+ .e_score_correction_bias as the gate bias when the layer has one),
              ....mlp.experts.<e>.gate_proj|up_proj|down_proj.weight (= w1, w3, w2),
              ....mlp.shared_experts.gate_proj|up_proj|down_proj.weight of width Es*H, cut into Es experts
              (the sum of Es SwiGLU experts is one SwiGLU MLP over the concatenated hidden units),
              model.layers.<i>.post_attention_layernorm.weight
In the "omega" scheme an expert (routed, shared or the dense one) may also come in the fused form of DiTSwiGLUFFN
(J/engine/nn/layer/dit/org/DiTSwiGLUFFN.java:79,127-141,296-303): "....w12.weight" [2H, d], whose first H rows are
the branch that goes through SiLU (channel 0 of the [number, 2, 1, H] view, this layer's w1) and whose last H rows
are the multiplier (channel 1, this layer's w3); the down projection then carries that class's name "....w3.weight"
and has shape [d, H].
Qwen-MoE checkpoints use the "deepseek" expert names; their sigmoid-gated shared expert is not part of this layer
and is refused.
"""
import json

import numpy as np

SCHEMES = ("omega", "mixtral", "deepseek")


def read_weight_map(path):
    """The whole file as {name: nested lists} (readJsonFileSmallWeight)."""
    with open(path, "r", encoding="utf-8") as f:
        m = json.load(f)
    if not isinstance(m, dict):
        raise RuntimeError("Error code 1:weight file is not a JSON object of name -> values")
    return m


def _tensor(meta, shape, key):
    """loadData: nested lists -> float32 row-major of the expected shape (1-D or 2-D); shape mismatches raise."""
    a = np.asarray(meta, dtype=np.float64)
    if a.shape != tuple(shape):
        raise RuntimeError(f"Error code 1:the tensor shape{list(shape)} is not shape:{list(a.shape)} ({key})")
    return np.ascontiguousarray(a.astype(np.float32))


def _names(scheme, i):
    if scheme == "omega":
        p = f"layers.{i}.feed_forward."
        return dict(gate=p + "gate.weight", gate_bias=p + "gate.bias", norm=f"layers.{i}.ffn_norm.weight",
                    expert=lambda e, w: f"{p}experts.{e}.{w}.weight",
                    shared=lambda s, w: f"{p}shared_experts.{s}.{w}.weight", dense=lambda w: f"{p}{w}.weight",
                    fused_shared=None)
    if scheme == "mixtral":
        p = f"model.layers.{i}.block_sparse_moe."
        return dict(gate=p + "gate.weight", gate_bias=None, norm=f"model.layers.{i}.post_attention_layernorm.weight",
                    expert=lambda e, w: f"{p}experts.{e}.{w}.weight", shared=None, dense=None, fused_shared=None)
    if scheme == "deepseek":
        p = f"model.layers.{i}.mlp."
        proj = {"w1": "gate_proj", "w3": "up_proj", "w2": "down_proj"}
        return dict(gate=p + "gate.weight", gate_bias=p + "gate.e_score_correction_bias",
                    norm=f"model.layers.{i}.post_attention_layernorm.weight",
                    expert=lambda e, w: f"{p}experts.{e}.{proj[w]}.weight", shared=None, dense=None,
                    fused_shared=lambda w: f"{p}shared_experts.{proj[w]}.weight")
    raise ValueError(f"unknown scheme {scheme!r}; one of {SCHEMES}")


def load_moe_weights(layer, weight_map, layer_index=0, scheme="omega", strict=True):
    """Copies the entries of `weight_map` (a dict as read_weight_map returns, or a path) that belong to layer
    `layer_index` into `layer` (anything with embedDim, hidden, nExperts, nShared, hasBias, set_gate, set_expert,
    set_norm).  Returns the list of expected names that were absent; with strict=True (default) an absent
    expert or gate weight raises instead (the reference reports "<key> is null." and goes on; a layer with
    unset experts is never what the caller wants).  The norm weight is optional: it belongs to the block form."""
    if isinstance(weight_map, (str, bytes)):
        weight_map = read_weight_map(weight_map)
    nm = _names(scheme, layer_index)
    d, H, E, Es = layer.embedDim, layer.hidden, layer.nExperts, layer.nShared
    missing = []

    def get(key, shape):
        if key is None or key not in weight_map:
            missing.append(key)
            return None
        return _tensor(weight_map[key], shape, key)

    if any(k.startswith(f"model.layers.{layer_index}.mlp.shared_expert_gate") for k in weight_map):
        raise RuntimeError("Error code 1:sigmoid-gated shared expert (shared_expert_gate) is not supported by this layer")
    Wg = get(nm["gate"], (E, d))
    bg = None
    if layer.hasBias and nm["gate_bias"] is not None:
        bg = get(nm["gate_bias"], (E,))
    if Wg is not None:
        layer.set_gate(Wg, bg)
    def one_expert(key):
        """(W1, W3, W2) of the expert whose parameter names key(w) gives, from the separate or the fused form."""
        if scheme == "omega" and key("w12") in weight_map:
            F, W2 = get(key("w12"), (2 * H, d)), get(key("w3"), (d, H))
            if F is None or W2 is None:
                return None
            return np.ascontiguousarray(F[:H]), np.ascontiguousarray(F[H:]), W2
        W1, W3, W2 = get(key("w1"), (H, d)), get(key("w3"), (H, d)), get(key("w2"), (d, H))
        return None if W1 is None or W3 is None or W2 is None else (W1, W3, W2)

    dense = (nm["dense"] is not None and E == 1 and nm["expert"](0, "w1") not in weight_map
             and nm["expert"](0, "w12") not in weight_map)
    for e in range(E):
        got = one_expert((lambda w: nm["dense"](w)) if dense else (lambda w, e=e: nm["expert"](e, w)))
        if got is not None:
            layer.set_expert(e, *got)
    if Es > 0:
        if nm["fused_shared"] is not None:
            F1, F3 = get(nm["fused_shared"]("w1"), (Es * H, d)), get(nm["fused_shared"]("w3"), (Es * H, d))
            F2 = get(nm["fused_shared"]("w2"), (d, Es * H))
            if F1 is not None and F3 is not None and F2 is not None:
                for s in range(Es):
                    layer.set_expert(E + s, np.ascontiguousarray(F1[s * H:(s + 1) * H]),
                                     np.ascontiguousarray(F3[s * H:(s + 1) * H]),
                                     np.ascontiguousarray(F2[:, s * H:(s + 1) * H]))
        elif nm["shared"] is not None:
            for s in range(Es):
                got = one_expert(lambda w, s=s: nm["shared"](s, w))
                if got is not None:
                    layer.set_expert(E + s, *got)
        else:
            raise RuntimeError(f"Error code 1:scheme {scheme!r} has no names for shared experts")
    required_missing = list(missing)
    if nm["norm"] in weight_map:
        layer.set_norm(_tensor(weight_map[nm["norm"]], (d,), nm["norm"]))
    else:
        missing.append(nm["norm"])
    if strict and required_missing:
        raise RuntimeError("Error code 1:" + ", ".join(f"{k} is null." for k in required_missing))
    return missing


def export_moe_weights(arrays, layer_index=0, scheme="omega", gamma=None, fused12=False):
    """The inverse, for tests and for exporting a layer: arrays = dict(Wg [E,d], bg [E]|None, W1,W3 [E+Es,H,d],
    W2 [E+Es,d,H]) -> {name: nested lists}.  fused12 ("omega" only): every expert in the DiTSwiGLUFFN form, w12 =
    [w1; w3] and the down projection under the name w3."""
    if fused12 and scheme != "omega":
        raise ValueError("fused12 belongs to the omega scheme")
    nm = _names(scheme, layer_index)
    E = arrays["Wg"].shape[0]
    G = arrays["W1"].shape[0]
    out = {nm["gate"]: arrays["Wg"].tolist()}
    if arrays.get("bg") is not None and nm["gate_bias"] is not None:
        out[nm["gate_bias"]] = arrays["bg"].tolist()
    def put(key, g):
        if fused12:
            out[key("w12")] = np.concatenate([arrays["W1"][g], arrays["W3"][g]], axis=0).tolist()
            out[key("w3")] = arrays["W2"][g].tolist()
        else:
            for w in ("w1", "w3", "w2"):
                out[key(w)] = arrays["W" + w[1]][g].tolist()

    for e in range(E):
        put(lambda w, e=e: nm["expert"](e, w), e)
    if G > E:
        if nm["fused_shared"] is not None:
            out[nm["fused_shared"]("w1")] = np.concatenate(list(arrays["W1"][E:]), axis=0).tolist()
            out[nm["fused_shared"]("w3")] = np.concatenate(list(arrays["W3"][E:]), axis=0).tolist()
            out[nm["fused_shared"]("w2")] = np.concatenate(list(arrays["W2"][E:]), axis=1).tolist()
        else:
            for s in range(G - E):
                put(lambda w, s=s: nm["shared"](s, w), E + s)
    if gamma is not None:
        out[nm["norm"]] = np.asarray(gamma).tolist()
    return out

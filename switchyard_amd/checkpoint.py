"""Reads an OLMoE checkpoint (Hugging Face layout: config.json plus one safetensors file or a
sharded set with model.safetensors.index.json) into the tensors the decoder and the MoE
kernels take.

Counterpart of the reference's switchyard/weights.py (:15-69) and switchyard/config.py
(:27-48): the same dictionary comes back, {"embed", "final_norm", "lm_head", "layers": [one
dict per layer], "experts"}, with a layer's experts stacked as gate_up [E, 2I, H] (gate rows
0..I-1, up rows I..2I-1) and down [E, H, I], each in nn.Linear layout (out x in, the reduced
dimension contiguous). That is the layout the kernels stream, so nothing is transposed or
repacked on the way in.

Built for a GPU that holds the whole model: every stacked tensor is allocated once on the
target device and each expert's matrices are copied from the file's mapping straight into
their rows of it, so the host never holds a second copy of a layer (a layer of OLMoE-1B-7B is
805 MB of experts; the reference stacks 128 host tensors per layer and then moves the stack).
Files are read with safetensors only: nothing in a checkpoint is executed.
"""

import json
import os

import torch
from safetensors import safe_open

from .decoder import Shape

INDEX = "model.safetensors.index.json"
SINGLE = "model.safetensors"


def shape_from_config(path):
    """The decoder's Shape from `path`/config.json (reference: Config.load, config.py:27-48).
    Returns (shape, tie_embeddings)."""
    with open(os.path.join(path, "config.json")) as f:
        c = json.load(f)
    heads = c["num_attention_heads"]
    rope = c.get("rope_parameters") or {}
    shape = Shape(vocab=c["vocab_size"], hidden=c["hidden_size"], intermediate=c["intermediate_size"],
                  layers=c["num_hidden_layers"], heads=heads, kv_heads=c.get("num_key_value_heads") or heads,
                  head_dim=c.get("head_dim") or c["hidden_size"] // heads, experts=c["num_experts"],
                  top_k=c["num_experts_per_tok"], norm_topk_prob=bool(c.get("norm_topk_prob", False)),
                  rms_eps=c.get("rms_norm_eps", 1e-5), rope_theta=rope.get("rope_theta", c.get("rope_theta", 10000.0)),
                  clip_qkv=c.get("clip_qkv"))
    return shape, bool(c.get("tie_word_embeddings", False))


class Checkpoint:
    """Name -> tensor over the files of one checkpoint directory; files are opened on first use
    and stay mapped until close()."""

    def __init__(self, path):
        self.path = path
        index = os.path.join(path, INDEX)
        if os.path.exists(index):
            with open(index) as f:
                self.where = dict(json.load(f)["weight_map"])
        elif os.path.exists(os.path.join(path, SINGLE)):
            with safe_open(os.path.join(path, SINGLE), "pt") as f:
                self.where = {k: SINGLE for k in f.keys()}
        else:
            raise FileNotFoundError(f"{path}: neither {INDEX} nor {SINGLE}")
        self._open = {}

    def has(self, name):
        return name in self.where

    def get(self, name):
        if name not in self.where:
            raise KeyError(f"{self.path}: no tensor named {name}")
        file = self.where[name]
        if file not in self._open:
            self._open[file] = safe_open(os.path.join(self.path, file), "pt")
        return self._open[file].get_tensor(name)

    def close(self):
        self._open.clear()


def load(path, shape=None, dtype=torch.float16, device="cuda", experts=None, experts_per_layer=None):
    """The weights of the checkpoint at `path` on `device` in `dtype`.

    `experts` (default: all) picks which experts are stacked, in that order; with
    `experts_per_layer`, layer i stacks experts_per_layer[i] instead (reference:
    weights.load, weights.py:36-69). The router keeps all its rows either way.
    Both the per-expert tensor names of published OLMoE checkpoints
    (`mlp.experts.<j>.gate_proj.weight` ...) and the stacked names newer transformers keeps in
    memory (`mlp.experts.gate_up_proj`, `mlp.experts.down_proj`) are understood."""
    tied = False
    if shape is None:
        shape, tied = shape_from_config(path)
    elif os.path.exists(os.path.join(path, "config.json")):
        tied = shape_from_config(path)[1]
    ck = Checkpoint(path)
    experts = list(range(shape.experts)) if experts is None else [int(e) for e in experts]
    if experts_per_layer is not None and len(experts_per_layer) != shape.layers:
        raise ValueError(f"experts_per_layer has {len(experts_per_layer)} entries for {shape.layers} layers")
    I, H = shape.intermediate, shape.hidden

    def t(name, want=None):
        x = ck.get(name)
        if want is not None and tuple(x.shape) != tuple(want):
            raise ValueError(f"{name}: shape {tuple(x.shape)} in the file, {tuple(want)} by config.json")
        return x.to(device=device, dtype=dtype).contiguous()

    def into(dst, name):
        x = ck.get(name)
        if tuple(x.shape) != tuple(dst.shape):
            raise ValueError(f"{name}: shape {tuple(x.shape)} in the file, {tuple(dst.shape)} by config.json")
        dst.copy_(x)          # converts and crosses to the device in one step, into the stack's own rows

    qd, kvd = shape.heads * shape.head_dim, shape.kv_heads * shape.head_dim
    out = {"embed": t("model.embed_tokens.weight", (shape.vocab, H)), "final_norm": t("model.norm.weight", (H,))}
    out["lm_head"] = out["embed"] if tied or not ck.has("lm_head.weight") else t("lm_head.weight", (shape.vocab, H))
    layers = []
    for i in range(shape.layers):
        p = f"model.layers.{i}."
        mine = experts if experts_per_layer is None else [int(e) for e in experts_per_layer[i]]
        bad = [e for e in mine if not 0 <= e < shape.experts]
        if bad:
            raise ValueError(f"layer {i}: experts {bad} outside 0..{shape.experts - 1}")
        gate_up = torch.empty(len(mine), 2 * I, H, dtype=dtype, device=device)
        down = torch.empty(len(mine), H, I, dtype=dtype, device=device)
        e = p + "mlp.experts."
        if ck.has(e + "gate_up_proj"):
            pick = torch.tensor(mine, dtype=torch.long)
            gate_up.copy_(ck.get(e + "gate_up_proj")[pick])
            down.copy_(ck.get(e + "down_proj")[pick])
        else:
            for row, j in enumerate(mine):
                into(gate_up[row, :I], f"{e}{j}.gate_proj.weight")
                into(gate_up[row, I:], f"{e}{j}.up_proj.weight")
                into(down[row], f"{e}{j}.down_proj.weight")
        layers.append(dict(
            attn_norm=t(p + "input_layernorm.weight", (H,)), mlp_norm=t(p + "post_attention_layernorm.weight", (H,)),
            wq=t(p + "self_attn.q_proj.weight", (qd, H)), wk=t(p + "self_attn.k_proj.weight", (kvd, H)),
            wv=t(p + "self_attn.v_proj.weight", (kvd, H)), wo=t(p + "self_attn.o_proj.weight", (H, qd)),
            q_norm=t(p + "self_attn.q_norm.weight", (qd,)), k_norm=t(p + "self_attn.k_norm.weight", (kvd,)),
            router=t(p + "mlp.gate.weight", (shape.experts, H)), gate_up=gate_up, down=down))
    ck.close()
    out["layers"] = layers
    out["experts"] = experts
    return out

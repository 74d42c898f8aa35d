"""Reads an OLMoE checkpoint (Hugging Face layout: config.json plus one safetensors file or a
sharded set with model.safetensors.index.json) into the tensors the decoder and the MoE
kernels take.

It fills the role of the reference's switchyard/weights.py (:36-69) and switchyard/config.py
(:27-48) and returns the same dictionary, {"embed", "final_norm", "lm_head", "layers": [one
dict per layer], "experts"}, with a layer's experts stacked as gate_up [E, 2I, H] (gate rows
0..I-1, up rows I..2I-1) and down [E, H, I], each in nn.Linear layout (out x in, the reduced
dimension contiguous). That is the layout the kernels stream, so nothing is transposed or
repacked on the way in.

The reader is destination-driven and makes one pass over the files. Every output tensor is
allocated on the target device first; a table then says, for each tensor name a checkpoint may
hold, which slice of which output it belongs in. The files are visited one after the other,
each opened once and closed again, and every tensor with an entry in the table is copied from
the file's mapping straight into its slice (the copy converts the type and crosses to the
device), so the host never holds a second copy of anything: a layer of OLMoE-1B-7B is 805 MB
of experts. Tensors without an entry (experts that were not asked for) are never read. Files
are read with safetensors only: nothing in a checkpoint is executed.
"""

import json
import os
from types import SimpleNamespace

import torch
from safetensors import safe_open

from .decoder import Shape

INDEX = "model.safetensors.index.json"
SINGLE = "model.safetensors"


def shape_from_config(path):
    """(Shape, tie_word_embeddings) from `path`/config.json; the field names are those of a
    transformers OlmoeConfig, which Shape.from_hf reads."""
    with open(os.path.join(path, "config.json")) as f:
        fields = json.load(f)
    return Shape.from_hf(SimpleNamespace(**fields)), bool(fields.get("tie_word_embeddings", False))


def tensor_files(path):
    """{file name: [tensor names in it]} for the checkpoint directory `path`."""
    index = os.path.join(path, INDEX)
    files = {}
    if os.path.exists(index):
        with open(index) as f:
            for name, file in json.load(f)["weight_map"].items():
                files.setdefault(file, []).append(name)
    elif os.path.exists(os.path.join(path, SINGLE)):
        with safe_open(os.path.join(path, SINGLE), "pt") as f:
            files[SINGLE] = list(f.keys())
    else:
        raise FileNotFoundError(f"{path}: neither {INDEX} nor {SINGLE}")
    return files


class _Slot:
    """Where one checkpoint tensor goes: `out` is the slice of an output tensor it fills; with
    `rows`, the tensor in the file is a stack and only those rows of it are taken."""

    def __init__(self, out, rows=None):
        self.out, self.rows, self.filled = out, rows, False

    def fill(self, name, get):
        x = get(name)
        want = tuple(self.out.shape[1:]) if self.rows is not None else tuple(self.out.shape)
        have = tuple(x.shape[1:]) if self.rows is not None else tuple(x.shape)
        if have != want or (self.rows is not None and max(self.rows, default=-1) >= x.shape[0]):
            raise ValueError(f"{name}: shape {tuple(x.shape)} in the file, {want} "
                             f"{'per expert ' if self.rows is not None else ''}by config.json")
        self.out.copy_(x if self.rows is None else x[torch.tensor(self.rows, dtype=torch.long)])
        self.filled = True


def _expert_lists(shape, experts, experts_per_layer):
    experts = list(range(shape.experts)) if experts is None else [int(e) for e in experts]
    if experts_per_layer is None:
        per_layer = [experts] * shape.layers
    elif len(experts_per_layer) != shape.layers:
        raise ValueError(f"experts_per_layer has {len(experts_per_layer)} entries for {shape.layers} layers")
    else:
        per_layer = [[int(e) for e in mine] for mine in experts_per_layer]
    for i, mine in enumerate(per_layer):
        bad = [e for e in mine if not 0 <= e < shape.experts]
        if bad:
            raise ValueError(f"layer {i}: experts {bad} outside 0..{shape.experts - 1}")
    return experts, per_layer


def load(path, shape=None, dtype=torch.float16, device="cuda", experts=None, experts_per_layer=None):
    """The weights of the checkpoint at `path` on `device` in `dtype`.

    `experts` (default: all) picks which experts are stacked, in that order; with
    `experts_per_layer`, layer i stacks experts_per_layer[i] instead (the arguments of the
    reference's weights.load, weights.py:36-38). The router keeps all its rows either way.
    Both the per-expert tensor names of published OLMoE checkpoints
    (`mlp.experts.<j>.gate_proj.weight` ...) and the stacked names newer transformers keeps in
    memory (`mlp.experts.gate_up_proj`, `mlp.experts.down_proj`) are understood."""
    tied = False
    if shape is None:
        shape, tied = shape_from_config(path)
    elif os.path.exists(os.path.join(path, "config.json")):
        tied = shape_from_config(path)[1]
    experts, per_layer = _expert_lists(shape, experts, experts_per_layer)
    files = tensor_files(path)
    present = {name for names in files.values() for name in names}
    H, I = shape.hidden, shape.intermediate
    qd, kvd = shape.heads * shape.head_dim, shape.kv_heads * shape.head_dim

    def new(*dims):
        return torch.empty(*dims, dtype=dtype, device=device)

    # ---- every output, and the table from checkpoint names to their places in them
    slots = {}
    out = {"embed": new(shape.vocab, H), "final_norm": new(H), "layers": [], "experts": experts}
    slots["model.embed_tokens.weight"] = _Slot(out["embed"])
    slots["model.norm.weight"] = _Slot(out["final_norm"])
    if tied or "lm_head.weight" not in present:
        out["lm_head"] = out["embed"]
    else:
        out["lm_head"] = new(shape.vocab, H)
        slots["lm_head.weight"] = _Slot(out["lm_head"])
    plain = (("attn_norm", "input_layernorm.weight", (H,)), ("mlp_norm", "post_attention_layernorm.weight", (H,)),
             ("wq", "self_attn.q_proj.weight", (qd, H)), ("wk", "self_attn.k_proj.weight", (kvd, H)),
             ("wv", "self_attn.v_proj.weight", (kvd, H)), ("wo", "self_attn.o_proj.weight", (H, qd)),
             ("q_norm", "self_attn.q_norm.weight", (qd,)), ("k_norm", "self_attn.k_norm.weight", (kvd,)),
             ("router", "mlp.gate.weight", (shape.experts, H)))
    for i, mine in enumerate(per_layer):
        prefix = f"model.layers.{i}."
        layer = {key: new(*dims) for key, _, dims in plain}
        layer["gate_up"], layer["down"] = new(len(mine), 2 * I, H), new(len(mine), H, I)
        for key, suffix, _ in plain:
            slots[prefix + suffix] = _Slot(layer[key])
        stacked = prefix + "mlp.experts.gate_up_proj"
        if stacked in present:   # one tensor holds all experts: take the rows asked for
            slots[stacked] = _Slot(layer["gate_up"], rows=mine)
            slots[prefix + "mlp.experts.down_proj"] = _Slot(layer["down"], rows=mine)
        else:
            for row, j in enumerate(mine):
                # the same expert may be stacked twice; each row is a place of its own
                for part, view in (("gate_proj", layer["gate_up"][row, :I]), ("up_proj", layer["gate_up"][row, I:]),
                                   ("down_proj", layer["down"][row])):
                    slots.setdefault(f"{prefix}mlp.experts.{j}.{part}.weight", []).append(_Slot(view))
        out["layers"].append(layer)

    # ---- one pass over the files
    for file, names in files.items():
        wanted = [name for name in names if name in slots]
        if not wanted:
            continue
        with safe_open(os.path.join(path, file), "pt") as f:
            for name in wanted:
                places = slots[name]
                for slot in places if isinstance(places, list) else [places]:
                    slot.fill(name, f.get_tensor)
    for name, places in slots.items():
        for slot in places if isinstance(places, list) else [places]:
            if not slot.filled:
                raise KeyError(f"{path}: no tensor named {name}")
    return out

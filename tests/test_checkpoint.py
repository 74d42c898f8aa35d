"""The checkpoint reader returns, from files written by transformers, the tensors its
in-memory state dict holds (bit for bit, stacked in the kernels' layout), and a decoder built
on them computes transformers' logits. Mirrors the reference's tests/test_model.py:19-34,86-94
(load from a tiny checkpoint on disk; loading a subset of experts)."""

import json
import os

import pytest
import torch
from safetensors.torch import save_file

from switchyard_amd import checkpoint as C
from switchyard_amd import decoder as D
from test_decoder import loop_hook, prompts, tiny

tr = pytest.importorskip("transformers")


def written(tmp_path, variant="plain", shard=None):
    hf, shape, weights = tiny(variant)
    path = str(tmp_path / variant)
    hf.save_pretrained(path, **({"max_shard_size": shard} if shard else {}))
    return path, hf, shape, weights


def same(a, b):
    assert a.keys() - {"experts"} == b.keys() - {"experts"}
    for k in ("embed", "final_norm", "lm_head"):
        assert torch.equal(a[k], b[k]), k
    for La, Lb in zip(a["layers"], b["layers"]):
        assert La.keys() == Lb.keys()
        for k in La:
            assert La[k].is_contiguous() and torch.equal(La[k], Lb[k]), k


@pytest.mark.parametrize("shard", [None, "100KB"])
def test_tensors_equal_the_state_dict(tmp_path, shard):
    path, hf, shape, weights = written(tmp_path, shard=shard)
    assert os.path.exists(os.path.join(path, C.INDEX)) == (shard is not None)
    got_shape, tied = C.shape_from_config(path)
    assert got_shape == shape and tied is False
    got = C.load(path, dtype=torch.float32, device="cpu")
    same(got, weights)
    assert got["experts"] == list(range(shape.experts))
    L = got["layers"][0]
    assert L["gate_up"].shape == (shape.experts, 2 * shape.intermediate, shape.hidden)
    assert L["down"].shape == (shape.experts, shape.hidden, shape.intermediate)


@pytest.mark.parametrize("variant", ["plain", "norm_topk", "gqa", "clip_qkv", "top4_of_16"])
def test_logits_from_a_checkpoint_match_transformers(tmp_path, variant):
    path, hf, _, _ = written(tmp_path, variant)
    shape, _ = C.shape_from_config(path)
    weights = C.load(path, shape, dtype=torch.float32, device="cpu")
    m = D.Decoder(shape, weights, moe=loop_hook(shape, weights), max_positions=256)
    for p in prompts(3):
        t = torch.tensor([p])
        with torch.no_grad():
            want = hf(t).logits
        assert (m.forward(t) - want).abs().max().item() < 1e-4


def test_loading_a_subset_of_experts(tmp_path):
    path, _, shape, _ = written(tmp_path)
    full = C.load(path, dtype=torch.float32, device="cpu")
    part = C.load(path, dtype=torch.float32, device="cpu", experts=[4, 5, 6, 7])
    assert part["experts"] == [4, 5, 6, 7]
    for L, P in zip(full["layers"], part["layers"]):
        assert torch.equal(L["gate_up"][4:], P["gate_up"]) and torch.equal(L["down"][4:], P["down"])
        assert torch.equal(L["router"], P["router"])
    per = C.load(path, dtype=torch.float32, device="cpu", experts_per_layer=[[7, 0], [3]])
    assert torch.equal(per["layers"][0]["gate_up"], full["layers"][0]["gate_up"][[7, 0]])
    assert torch.equal(per["layers"][1]["down"], full["layers"][1]["down"][[3]])
    with pytest.raises(ValueError):
        C.load(path, dtype=torch.float32, device="cpu", experts=[shape.experts])
    with pytest.raises(ValueError):
        C.load(path, dtype=torch.float32, device="cpu", experts_per_layer=[[0]])


def test_stacked_names_tied_embeddings_and_conversion(tmp_path):
    """A file that keeps the experts stacked (the names transformers holds in memory) and has
    no lm_head reads to the same tensors; lm_head is then the embedding; dtype converts once."""
    path, hf, shape, weights = written(tmp_path)
    sd = {k: v.contiguous() for k, v in hf.state_dict().items() if k != "lm_head.weight"}
    assert any(k.endswith("mlp.experts.gate_up_proj") for k in sd)
    stacked = str(tmp_path / "stacked")
    os.makedirs(stacked)
    save_file(sd, os.path.join(stacked, C.SINGLE))
    cfg = json.load(open(os.path.join(path, "config.json")))
    cfg["tie_word_embeddings"] = True
    json.dump(cfg, open(os.path.join(stacked, "config.json"), "w"))
    got = C.load(stacked, dtype=torch.float32, device="cpu", experts=[2, 5])
    assert got["lm_head"] is got["embed"]
    for L, W in zip(got["layers"], weights["layers"]):
        assert torch.equal(L["gate_up"], W["gate_up"][[2, 5]]) and torch.equal(L["down"], W["down"][[2, 5]])
    half = C.load(path, dtype=torch.float16, device="cpu")
    assert half["layers"][1]["down"].dtype == torch.float16
    assert torch.equal(half["layers"][1]["down"], weights["layers"][1]["down"].half())


def test_errors_name_the_file_and_the_tensor(tmp_path):
    with pytest.raises(FileNotFoundError):
        C.tensor_files(str(tmp_path))
    path, _, shape, _ = written(tmp_path)
    wrong = D.Shape(**{**shape.__dict__, "intermediate": shape.intermediate * 2})
    with pytest.raises(ValueError, match=r"experts\.\d+\.(gate|up|down)_proj"):
        C.load(path, wrong, dtype=torch.float32, device="cpu")
    with pytest.raises(KeyError, match="layers.2"):
        C.load(path, D.Shape(**{**shape.__dict__, "layers": 3}), dtype=torch.float32, device="cpu")


@pytest.mark.gpu
def test_a_checkpoint_loads_onto_the_gpu_and_decodes_through_the_kernels(tmp_path):
    """fp16 on the GPU, experts copied straight into the stacked device tensors: the default
    hook (HIP kernels) gives the logits of the per-expert loop on the same loaded weights."""
    torch.manual_seed(3)
    cfg = tr.OlmoeConfig(vocab_size=500, hidden_size=256, intermediate_size=128, num_hidden_layers=2,
                         num_attention_heads=4, num_key_value_heads=4, num_experts=64, num_experts_per_tok=8,
                         max_position_embeddings=128, eos_token_id=1, pad_token_id=0, bos_token_id=2)
    hf = tr.OlmoeForCausalLM(cfg).eval()
    with torch.no_grad():
        for name, p in hf.named_parameters():
            if "norm" not in name:
                p.normal_(0, 0.05)
    path = str(tmp_path / "ck")
    hf.save_pretrained(path, max_shard_size="2MB")
    w = C.load(path)
    shape, _ = C.shape_from_config(path)
    assert w["layers"][0]["gate_up"].is_cuda and w["layers"][0]["gate_up"].dtype == torch.float16
    assert torch.equal(w["layers"][1]["down"][5].cpu(),
                       hf.state_dict()["model.layers.1.mlp.experts.down_proj"][5].half())
    t = torch.randint(3, 500, (3, 20), generator=torch.Generator().manual_seed(0)).cuda()
    fast = D.Decoder(shape, w, max_positions=128).forward(t)
    slow = D.Decoder(shape, w, moe=loop_hook(shape, w), max_positions=128).forward(t)
    assert (fast.float() - slow.float()).abs().max().item() < 2e-2

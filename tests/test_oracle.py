"""Pins the CPU oracle: the reference's known-answer test, library cross-checks, brute force,
an independent plain-C restatement and the transformers OLMoE block. Runs without a GPU."""

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import cases
from oracle import c_oracle
from oracle import moe_oracle as O


# ------------------------------------------------------------------ sort / plan
def test_plan_known_answer_from_the_reference_tests():
    # The literal vector of the reference's tests/test_model.py:49-57; pos_of by ep.py:40-41.
    g = cases.golden_sort_vector()
    p = O.plan(torch.tensor(g["idx"]), torch.tensor(g["w"]), g["n_experts"])
    assert p.counts.tolist() == g["counts"]
    assert p.offsets.tolist() == g["offsets"]
    assert p.token.tolist() == g["token"]
    assert p.slot.tolist() == g["slot"]
    assert torch.allclose(p.weight, torch.tensor(g["weight"]))
    assert p.pos_of.tolist() == g["pos_of"]


def test_c_sort_known_answer_from_the_reference_tests():
    g = cases.golden_sort_vector()
    counts, offsets, token, wsorted, pos_of = c_oracle.sort_by_expert(
        np.array(g["idx"], dtype=np.int32), np.array(g["w"], dtype=np.float32), g["n_experts"])
    assert counts.tolist() == g["counts"]
    assert offsets.tolist() == g["offsets"]
    assert token.tolist() == g["token"]
    assert np.allclose(wsorted, g["weight"])
    assert pos_of.tolist() == g["pos_of"]


@pytest.mark.parametrize("N,k,E", [(1, 8, 64), (37, 8, 64), (300, 4, 60), (64, 2, 8), (500, 8, 128), (5, 3, 200)])
def test_plan_invariants_and_c_restatement_agree(N, k, E):
    g = torch.Generator().manual_seed(N * 131 + E)
    # distinct experts per token, in random slot order
    idx = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(N)])
    w = torch.rand(N, k, generator=g).half()
    p = O.plan(idx, w, E)
    M = N * k
    assert int(p.offsets[-1]) == M and int(p.counts.sum()) == M
    assert torch.equal(p.counts, torch.bincount(idx.flatten(), minlength=E))
    for e in range(E):
        seg = p.token[p.offsets[e]:p.offsets[e + 1]]
        assert torch.all(seg[1:] >= seg[:-1])                      # token order inside an expert
    assert sorted(p.pos_of.tolist()) == list(range(M))             # a permutation
    assert torch.equal(p.token[p.pos_of], torch.arange(M) // k)
    row_expert = torch.repeat_interleave(torch.arange(E), p.counts)
    assert torch.equal(row_expert[p.pos_of], idx.flatten())
    c = c_oracle.sort_by_expert(idx.numpy(), w.numpy(), E)
    assert np.array_equal(c[0], p.counts.numpy()) and np.array_equal(c[1], p.offsets.numpy())
    assert np.array_equal(c[2], p.token.numpy()) and np.array_equal(c[4], p.pos_of.numpy())
    assert np.array_equal(c[3].view(np.uint16), p.weight.numpy().view(np.uint16))  # a pure permutation


def test_plan_with_repeated_experts_in_a_token_is_still_the_stable_sort():
    idx = torch.tensor([[1, 1, 0], [0, 1, 1]])
    w = torch.arange(6, dtype=torch.float32).view(2, 3)
    p = O.plan(idx, w, 2)
    assert p.token.tolist() == [0, 1, 0, 0, 1, 1] and p.slot.tolist() == [2, 0, 0, 1, 1, 2]
    c = c_oracle.sort_by_expert(idx.numpy(), w.numpy(), 2)
    assert c[2].tolist() == p.token.tolist() and c[4].tolist() == p.pos_of.tolist()


# ------------------------------------------------------------------ route
@pytest.mark.parametrize("E,k", [(8, 2), (64, 8), (60, 4), (128, 8), (16, 4)])
@pytest.mark.parametrize("norm", [False, True])
def test_route_equals_torch_topk_softmax_on_tie_free_rows(E, k, norm):
    g = torch.Generator().manual_seed(E + k)
    logits = torch.randn(400, E, generator=g)                      # fp32 noise: ties have measure ~0
    idx, w = O.route_logits(logits, k, norm)
    probs = torch.softmax(logits, -1, dtype=torch.float32)
    tw, tidx = torch.topk(probs, k, dim=-1)
    if norm:
        tw = tw / tw.sum(-1, keepdim=True)
    assert torch.equal(idx, tidx)
    assert torch.equal(w, tw)


def test_route_tie_rule_lower_expert_id_wins():
    logits = torch.tensor([[1.0, 3.0, 3.0, 0.5, 3.0, 1.0, 1.0, -2.0]])
    idx, w = O.route_logits(logits, 5, False)
    assert idx.tolist() == [[1, 2, 4, 0, 5]]
    cidx, cw = c_oracle.route(logits.numpy(), 5, False)
    assert cidx.tolist() == [[1, 2, 4, 0, 5]]
    assert np.allclose(cw, w.numpy(), atol=1e-7)
    assert O.brute_force_topk(logits[0].tolist(), 5) == [1, 2, 4, 0, 5]


@pytest.mark.parametrize("norm", [False, True])
def test_route_on_fp16_logits_with_many_ties_matches_c_and_brute_force(norm):
    # fp16 logits of the benchmark's scale: exact ties are common, some straddle the top-k edge
    g = torch.Generator().manual_seed(7)
    h = torch.randn(2048, 256, generator=g).half()
    router = (torch.randn(64, 256, generator=g) * 0.06).half()
    logits = F.linear(h.float(), router.float()).half()
    idx, w = O.route_logits(logits, 8, norm)
    cidx, cw = c_oracle.route(logits.float().numpy(), 8, norm)
    assert np.array_equal(idx.numpy().astype(np.int32), cidx)
    assert np.abs(w.float().numpy() - cw).max() < 1e-3
    srt = torch.sort(logits.float(), dim=-1, descending=True).values
    assert int((srt[:, 7] == srt[:, 8]).sum()) > 0                 # the tie rule is exercised
    for t in range(0, 2048, 97):
        assert O.brute_force_topk(logits[t].tolist(), 8) == idx[t].tolist()


def test_route_weights_are_softmax_values():
    g = torch.Generator().manual_seed(3)
    logits = torch.randn(50, 64, generator=g).half()
    idx, w = O.route_logits(logits, 8, False)
    p64 = torch.softmax(logits.double(), -1).gather(1, idx)
    assert (w.double() - p64).abs().max() < 1e-3
    idx2, w2 = O.route_logits(logits, 8, True)
    assert torch.equal(idx, idx2)
    assert (w2.float().sum(-1) - 1).abs().max() < 4e-3


# ------------------------------------------------------------------ experts
def _tiny(seed=0, E=8, H=16, I=12, N=40, k=3):
    torch.manual_seed(seed)
    h = torch.randn(N, H)
    router = torch.randn(E, H)
    gu, dn = torch.randn(E, 2 * I, H) * 0.3, torch.randn(E, H, I) * 0.3
    return h, router, gu, dn, k


def test_grouped_experts_equal_the_loop_bit_for_bit_in_fp32():
    # The reference's property test, tests/test_model.py:37-46.
    h, router, gu, dn, k = _tiny()
    idx, w = O.route(h, router, k, False)
    a = O.experts_loop(h, idx, w, gu, dn)
    b = O.experts_grouped(h, idx, w, gu, dn)
    assert torch.equal(a, b)


def test_loop_equals_float64_brute_force_and_scalar_c():
    h, router, gu, dn, k = _tiny(seed=1)
    idx, w = O.route(h, router, k, False)
    got = O.experts_loop(h, idx, w, gu, dn)
    want = O.brute_force_layer(h.numpy(), idx.numpy(), w.numpy(), gu.numpy(), dn.numpy())
    assert np.abs(got.double().numpy() - want).max() < 1e-5
    c = c_oracle.experts_f32(h.numpy(), idx.numpy(), w.numpy(), gu.numpy(), dn.numpy())
    assert np.abs(c.astype(np.float64) - want).max() < 1e-5


def test_gate_rows_come_first_in_gate_up():
    # a dropped or swapped half of gate_up changes the answer: silu(g)*u != silu(u)*g
    x = torch.tensor([[1.0, 2.0]])
    gate_up = torch.tensor([[1.0, 0.0], [0.0, 1.0]])              # gate = x0, up = x1
    down = torch.tensor([[1.0]])
    y = O.expert_mlp(x, gate_up, down)
    assert abs(float(y) - (1.0 / (1.0 + np.exp(-1.0))) * 2.0) < 1e-6


def test_ffn_rows_and_combine_rows_rebuild_the_loop():
    h, router, gu, dn, k = _tiny(seed=2)
    idx, w = O.route(h, router, k, False)
    p = O.plan(idx, w, gu.shape[0])
    y = O.ffn_rows(h, p.token, p.offsets, p.weight, gu, dn)
    out = O.combine_rows(y, p.pos_of, idx, h.shape[0])
    assert (out - O.experts_loop(h, idx, w, gu, dn)).abs().max() < 1e-5
    # combine_rows equals index_add_ of the sorted rows in row order (ep.py:48-55)
    ref = torch.zeros_like(h).index_add_(0, p.token, y)
    assert (out - ref).abs().max() < 1e-5
    # and its order is ascending expert id
    order = c_oracle.combine_order(idx.numpy())
    assert np.array_equal(order, torch.sort(idx, dim=1, stable=True).indices.numpy())


def test_tile_offsets_closed_form():
    counts = torch.tensor([0, 1, 64, 65, 128, 0, 200])
    assert O.tile_offsets(counts).tolist() == [0, 0, 1, 2, 4, 6, 6, 10]
    assert O.tile_offsets(counts, 128).tolist() == [0, 0, 1, 2, 3, 4, 4, 6]


# ------------------------------------------------------------------ an independent second source
@pytest.mark.parametrize("norm", [False, True])
def test_layer_matches_the_transformers_olmoe_block(norm):
    tr = pytest.importorskip("transformers")
    from transformers.models.olmoe.modeling_olmoe import OlmoeSparseMoeBlock

    torch.manual_seed(0)
    cfg = tr.OlmoeConfig(vocab_size=32, hidden_size=32, intermediate_size=24, num_hidden_layers=1,
                         num_attention_heads=2, num_key_value_heads=2, num_experts=16, num_experts_per_tok=4,
                         norm_topk_prob=norm)
    blk = OlmoeSparseMoeBlock(cfg).eval()
    with torch.no_grad():
        blk.gate.weight.normal_(0, 1.0)
        blk.experts.gate_up_proj.normal_(0, 0.2)
        blk.experts.down_proj.normal_(0, 0.2)
        x = torch.randn(2, 9, 32)
        want = blk(x)
        want = want[0] if isinstance(want, tuple) else want
        got = O.moe_layer(x.view(-1, 32), blk.gate.weight, blk.experts.gate_up_proj, blk.experts.down_proj, 4, norm)
    assert (got - want.reshape(-1, 32)).abs().max() < 1e-5


def test_config1_tiny_layer_runs_and_is_bit_stable():
    # hidden 128, intermediate 64, 16 experts, top-4, fp32, 32 tokens, weights N(0, 0.02)
    from cases import layer

    h, router, gu, dn = layer(32, E=16, k=4, H=128, I=64, seed=0, dtype=torch.float32)
    idx, w = O.route(h, router, 4, False)
    a = O.experts_loop(h, idx, w, gu, dn)
    b = O.experts_grouped(h, idx, w, gu, dn)
    assert torch.equal(a, b)
    cidx, _ = c_oracle.route(F.linear(h, router).numpy(), 4, False)
    assert np.array_equal(cidx, idx.numpy().astype(np.int32))
    want = O.brute_force_layer(h.numpy(), idx.numpy(), w.numpy(), gu.numpy(), dn.numpy())
    assert np.abs(a.double().numpy() - want).max() < 1e-6

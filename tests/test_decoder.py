"""The decoder harness around the MoE hook computes what transformers' OLMoE computes (CPU, fp32,
with the oracle's per-expert loop in the hook), and on a GPU the hook with the HIP kernels
decodes the same tokens as the hook with the fp16 per-expert loop."""

import pytest
import torch

from oracle import moe_oracle as O
from switchyard_amd import decoder as D

tr = pytest.importorskip("transformers")

VARIANTS = {
    "plain": {},
    "norm_topk": {"norm_topk_prob": True},
    "gqa": {"num_attention_heads": 4, "num_key_value_heads": 2},
    "clip_qkv": {"clip_qkv": 0.3},
    "top4_of_16": {"num_experts": 16, "num_experts_per_tok": 4},
}
_CACHE = {}


def tiny(variant):
    if variant in _CACHE:
        return _CACHE[variant]
    torch.manual_seed(0)
    kw = dict(vocab_size=131, hidden_size=64, intermediate_size=32, num_hidden_layers=2, num_attention_heads=4,
              num_key_value_heads=4, num_experts=8, num_experts_per_tok=2, max_position_embeddings=256,
              eos_token_id=1, pad_token_id=0, bos_token_id=2)
    kw.update(VARIANTS[variant])
    cfg = tr.OlmoeConfig(**kw)
    hf = tr.OlmoeForCausalLM(cfg).eval()
    with torch.no_grad():
        for name, p in hf.named_parameters():
            if "norm" in name:
                p.copy_(1.0 + 0.1 * torch.randn_like(p))
            elif "gate.weight" in name:
                p.normal_(0, 1.0)          # a spread-out router picks distinct experts
            else:
                p.normal_(0, 0.08)
    shape = D.Shape.from_hf(cfg)
    weights = D.weights_from_hf(hf.state_dict(), shape)
    _CACHE[variant] = (hf, shape, weights)
    return _CACHE[variant]


def loop_hook(shape, weights):
    def moe(i, h):
        L = weights["layers"][i]
        return O.moe_layer(h, L["router"], L["gate_up"], L["down"], shape.top_k, shape.norm_topk_prob)
    return moe


def prompts(n, vocab=131, seed=0):
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(3, vocab, (int(torch.randint(6, 24, (1,), generator=g)),), generator=g).tolist()
            for _ in range(n)]


@pytest.mark.parametrize("variant", VARIANTS)
def test_logits_match_transformers(variant):
    hf, shape, weights = tiny(variant)
    m = D.Decoder(shape, weights, moe=loop_hook(shape, weights), max_positions=256)
    for p in prompts(3):
        t = torch.tensor([p])
        with torch.no_grad():
            want = hf(t).logits
        assert (m.forward(t) - want).abs().max().item() < 1e-4


@pytest.mark.parametrize("variant", ["plain", "gqa"])
def test_decoding_with_the_cache_equals_a_full_forward(variant):
    _, shape, weights = tiny(variant)
    m = D.Decoder(shape, weights, moe=loop_hook(shape, weights), max_positions=256)
    p = prompts(1, seed=3)[0]
    full = m.forward(torch.tensor([p + [5, 6, 7]]))
    cache = D.KVCache(shape, 1, 40, torch.float32, "cpu")
    out = [m.forward(torch.tensor([p]), cache)]
    for t in (5, 6, 7):
        out.append(m.forward(torch.tensor([[t]]), cache))
    assert (torch.cat(out, 1) - full).abs().max().item() < 1e-4


def test_greedy_generation_matches_transformers_and_batching_changes_nothing():
    hf, shape, weights = tiny("plain")
    m = D.Decoder(shape, weights, moe=loop_hook(shape, weights), max_positions=256)
    ps = prompts(4, seed=5)
    batched = m.generate(ps, 10)
    for p, got in zip(ps, batched):
        alone = m.generate([p], 10)[0]
        with torch.no_grad():
            want = hf.generate(torch.tensor([p]), max_new_tokens=10, do_sample=False,
                               eos_token_id=None)[0, len(p):].tolist()
        assert got == alone == want


def test_generation_stops_after_eos():
    _, shape, weights = tiny("plain")
    m = D.Decoder(shape, weights, moe=loop_hook(shape, weights), max_positions=256)
    ps = prompts(3, seed=9)
    free = m.generate(ps, 12)
    eos = free[0][4]
    cut = m.generate(ps, 12, eos=eos)
    for a, b in zip(free, cut):
        assert b == (a[:a.index(eos) + 1] if eos in a else a)[:len(b)] and (eos not in b[:-1])


def test_random_weights_have_the_loader_layout():
    s = D.Shape(vocab=50, hidden=32, intermediate=16, layers=1, heads=2, kv_heads=2, head_dim=16, experts=4, top_k=2)
    w = D.random_weights(s, dtype=torch.float32, device="cpu")
    L = w["layers"][0]
    assert L["gate_up"].shape == (4, 32, 32) and L["down"].shape == (4, 32, 16) and L["router"].shape == (4, 32)
    assert w["embed"].shape == (50, 32) and w["lm_head"].shape == (50, 32)


@pytest.mark.gpu
@pytest.mark.parametrize("batch", [2, 8])
def test_kernel_hook_decodes_the_same_tokens_as_the_loop_hook(batch):
    """fp16 on the GPU: hook = HIP kernels against hook = per-expert loop (oracle) on the same
    weights. The first logits agree to 2e-2 with the same top-1; every token the kernels'
    greedy decode picks is the loop model's top-1 for the same prefix, up to ties inside the
    logits tolerance (a random-init model has near-equal logits, and the two hooks round their
    fp16 sums in different orders); where the loop model's margin is clear the pick is the same."""
    s = D.Shape(vocab=1000, hidden=512, intermediate=256, layers=4, heads=8, kv_heads=8, head_dim=64, experts=64, top_k=8)
    w = D.random_weights(s, device="cuda", seed=1, std=0.05)
    ps = [torch.randint(3, s.vocab, (24 + 3 * b,), generator=torch.Generator().manual_seed(b)).tolist()
          for b in range(batch)]
    fast = D.Decoder(s, w, max_positions=128)
    slow = D.Decoder(s, w, moe=loop_hook(s, w), max_positions=128)
    new = 16
    a, la = fast.generate(ps, new, return_first_logits=True)
    _, lb = slow.generate(ps, new, return_first_logits=True)
    tol = 2e-2
    assert (la.float() - lb.float()).abs().max().item() < tol
    clear = lb.float().topk(2, -1).values
    clear = (clear[:, 0] - clear[:, 1]) > 2 * tol
    assert torch.equal(la.argmax(-1)[clear], lb.argmax(-1)[clear])
    checked = 0  # positions with a clear margin (informational: a random-init model has few)
    for prompt, picked in zip(ps, a):
        seq = torch.tensor([prompt + picked], device="cuda")
        logits = slow.forward(seq)[0, len(prompt) - 1:len(prompt) - 1 + len(picked)].float()
        best = logits.max(-1).values
        chosen = logits.gather(1, torch.tensor(picked, device="cuda")[:, None])[:, 0]
        assert (best - chosen).max().item() <= 2 * tol, "a picked token is not the loop model's top-1 within tolerance"
        top2 = logits.topk(2, -1).values
        sure = (top2[:, 0] - top2[:, 1]) > 2 * tol
        assert torch.equal(logits.argmax(-1)[sure].cpu(), torch.tensor(picked)[sure.cpu()])
        checked += int(sure.sum())


@pytest.mark.gpu
def test_full_size_model_as_written_agrees_with_the_loop_hook():
    """The full-model configuration at its stated size: 16 layers of OLMoE-1B-7B's shape with
    random fp16 weights (about 14 GB), 8 prompts of 512 tokens, attention in PyTorch operators and
    the MoE layers through the hook -> kernels.moe_layer, the decode step replayed as a HIP graph.
    The first logits agree with the same model with the per-expert loop in the hook to 2e-2, every
    row's first token is that model's top-1 (exactly where its margin is clear of the tolerance),
    and the replayed steps decode what the eager steps decode."""
    s = D.OLMOE_1B_7B
    w = D.random_weights(s, device="cuda", seed=0)
    B, P, new = 8, 512, 8
    ps = torch.randint(3, s.vocab, (B, P), generator=torch.Generator().manual_seed(0)).tolist()
    fast = D.Decoder(s, w, max_positions=P + new + 8, attention="torch")
    slow = D.Decoder(s, w, moe=loop_hook(s, w), max_positions=P + new + 8, attention="torch")
    tokens, first = fast.generate_graph(ps, new, return_first_logits=True)
    ref = slow.forward(torch.tensor(ps, device="cuda"))[:, -1]
    tol = 2e-2
    assert (first.float() - ref.float()).abs().max().item() < tol
    top2 = ref.float().topk(2, -1).values
    clear = (top2[:, 0] - top2[:, 1]) > 2 * tol
    picked = first.argmax(-1)
    assert torch.equal(picked[clear], ref.argmax(-1)[clear])
    chosen = ref.float().gather(1, picked[:, None])[:, 0]
    assert (top2[:, 0] - chosen).max().item() <= 2 * tol, "a first token is not the loop model's top-1 within tolerance"
    assert [t[0] for t in tokens] == picked.tolist()
    assert fast.generate(ps, new) == tokens
    del fast, slow, w
    torch.cuda.empty_cache()


@pytest.mark.gpu
def test_graph_replayed_decode_equals_eager_decode():
    """The decode step captured in a HIP graph and replayed (with eager work between two
    generations) yields the tokens of the eager loop, every time."""
    s = D.Shape(vocab=1000, hidden=512, intermediate=256, layers=3, heads=8, kv_heads=8, head_dim=64, experts=64, top_k=8)
    w = D.random_weights(s, device="cuda", seed=2, std=0.05)
    m = D.Decoder(s, w, max_positions=128)
    ps = [torch.randint(3, s.vocab, (20 + 5 * b,), generator=torch.Generator().manual_seed(b)).tolist() for b in range(4)]
    eager = m.generate(ps, 12)
    for _ in range(3):
        assert m.generate_graph(ps, 12) == eager
        assert m.generate(ps, 12) == eager


def test_the_kernels_are_not_silently_replaced_on_the_cpu():
    """attention="kernels" on weights the kernels cannot take (CPU, fp32) raises; "auto" there
    means the PyTorch operators, and the default MoE hook has no CPU form at all."""
    _, shape, weights = tiny("plain")
    with pytest.raises(ValueError):
        D.Decoder(shape, weights, max_positions=64, attention="kernels")
    m = D.Decoder(shape, weights, max_positions=64)
    assert m.fused is False
    with pytest.raises(RuntimeError):
        m.forward(torch.tensor([[3, 4, 5]]))      # the default hook calls the HIP kernels: CPU tensors are refused

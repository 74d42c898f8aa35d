"""CPU oracle for the OLMoE mixture-of-experts layer. TEST INFRASTRUCTURE ONLY.

This module restates, on the CPU with torch/numpy library routines, the function that the
HIP kernels of `switchyard_amd` compute. It exists to check them. Only the test suite, the
smoke check and the CPU-baseline leg of the benchmark may import it; the product path never
does and fails loudly when its HIP library is missing.

Each function cites the reference source it follows (paths under the reference tree):

  route              switchyard/moe.py:17-25, tie rule switchyard/csrc/moe_kernels.cu:52,57
  plan               switchyard/moe.py:45-63, pos_of from switchyard/ep.py:38-42
  expert_mlp         switchyard/moe.py:28-31
  experts_loop       switchyard/moe.py:34-42   (the per-expert loop; also the CPU baseline)
  run_sorted         switchyard/moe.py:66-74
  combine            switchyard/moe.py:77-82
  experts_grouped    switchyard/moe.py:85-88
  experts_fp16_graph switchyard/kernels.py:64-73 + rounding points moe_kernels.cu:253-259
  combine_rows       switchyard/csrc/moe_kernels.cu:419-433 (fp32 sum in expert order)
  tile_offsets       switchyard/kernels.py:23-27

How each is pinned (tests/test_oracle.py): `plan` by the reference's own known-answer test
(tests/test_model.py:49-57) and by the C restatement in oracle/route_sort.c; `route` by
torch.topk(softmax) on tie-free rows, a brute-force scan and the C restatement;
`expert_mlp`/`experts_loop` by a float64 brute force over (token, slot) and by the
transformers OlmoeSparseMoeBlock; `experts_grouped` by bit-equality with the loop in fp32
(tests/test_model.py:37-46); `combine_rows` by index_add_ in row order (ep.py:48-55).

Tie rule. The reference kernel orders candidates by (exp(logit - max) descending, expert id
ascending); torch.topk leaves ties unspecified. exp is monotone, so this oracle orders by
(logit descending, expert id ascending), which is exactly defined on every platform. The two
keys can differ only where fp32 rounding of `logit - max` merges two distinct logits, a case
whose outcome in the reference depends on the platform's expf.
"""

from dataclasses import dataclass

import numpy as np
import torch
import torch.nn.functional as F


def route_logits(logits, top_k, norm_topk_prob, out_dtype=None):
    """logits [N, E] (any float dtype) -> (idx int64 [N, k], w [N, k]).

    Softmax in float32 over all experts, the k largest ordered by (logit desc, id asc),
    optional renormalisation over the chosen k, cast to `out_dtype` (default: logits' dtype).
    """
    lf = logits.float()
    probs = torch.softmax(lf, dim=-1)
    order = torch.sort(lf, dim=-1, descending=True, stable=True).indices
    idx = order[:, :top_k].contiguous()
    w = probs.gather(1, idx)
    if norm_topk_prob:
        w = w / w.sum(dim=-1, keepdim=True)
    return idx, w.to(out_dtype or logits.dtype)


def route(h, router, top_k, norm_topk_prob):
    """h [N, H], router [E, H] -> (idx int64 [N, k], w [N, k] in h's dtype)."""
    return route_logits(F.linear(h, router), top_k, norm_topk_prob, h.dtype)


def expert_mlp(x, gate_up, down):
    """SwiGLU expert: x [n, H], gate_up [2I, H] (gate rows first), down [H, I]."""
    gate, up = F.linear(x, gate_up).chunk(2, dim=-1)
    return F.linear(F.silu(gate) * up, down)


def experts_loop(h, idx, w, gate_up, down):
    """The per-expert loop: experts ascending, each adds its rows into `out` (h's dtype)."""
    out = torch.zeros_like(h)
    for e in range(gate_up.shape[0]):
        tok, slot = torch.where(idx == e)
        if tok.numel() == 0:
            continue
        y = expert_mlp(h[tok], gate_up[e], down[e]) * w[tok, slot, None]
        out.index_add_(0, tok, y.to(out.dtype))
    return out


@dataclass
class Plan:
    """Choices sorted by expert: row i is token[i]'s slot[i]-th choice; expert e owns rows
    offsets[e]:offsets[e+1]; pos_of[t*k+s] is the row of token t's s-th choice."""
    token: torch.Tensor
    slot: torch.Tensor
    weight: torch.Tensor
    counts: torch.Tensor
    offsets: torch.Tensor
    pos_of: torch.Tensor


def plan(idx, w, num_experts):
    """Stable sort of the flat choices i = t*k + s by expert id."""
    N, k = idx.shape
    flat = idx.reshape(-1).to(torch.int64)
    order = torch.sort(flat, stable=True).indices
    counts = torch.bincount(flat, minlength=num_experts)
    offsets = torch.zeros(num_experts + 1, dtype=torch.int64, device=idx.device)
    offsets[1:] = torch.cumsum(counts, 0)
    pos_of = torch.empty(flat.numel(), dtype=torch.int64, device=idx.device)
    pos_of[order] = torch.arange(flat.numel(), dtype=torch.int64, device=idx.device)
    return Plan(order // k, order % k, w.reshape(-1)[order], counts, offsets, pos_of)


def run_sorted(x_sorted, counts, gate_up, down):
    out = torch.empty(x_sorted.shape[0], down.shape[1], dtype=x_sorted.dtype, device=x_sorted.device)
    start = 0
    for e, n in enumerate(counts.tolist()):
        if n:
            out[start:start + n] = expert_mlp(x_sorted[start:start + n], gate_up[e], down[e])
        start += n
    return out


def combine(y_sorted, p, n_tokens):
    out = torch.zeros(n_tokens, y_sorted.shape[1], dtype=y_sorted.dtype, device=y_sorted.device)
    out.index_add_(0, p.token, y_sorted * p.weight[:, None])
    return out


def experts_grouped(h, idx, w, gate_up, down):
    p = plan(idx, w, gate_up.shape[0])
    y = run_sorted(h[p.token], p.counts, gate_up, down)
    return combine(y, p, h.shape[0])


def ffn_rows(x, a_rows, offsets, wsorted, gate_up, down):
    """Sorted rows through their experts, scaled by the router weight: the function the two
    grouped projections compute together. Row i reads x[a_rows[i]] (x[i] when a_rows is
    None). In fp16 every intermediate is rounded where the fp16 torch graph rounds it."""
    xs = x[a_rows.long()] if a_rows is not None else x
    counts = (offsets[1:] - offsets[:-1]).long()
    return run_sorted(xs, counts, gate_up, down) * wsorted[:, None]


def combine_rows(y, pos_of, idx, n_tokens):
    """out[t] = sum_j y[pos_of[t*k+j]] over t's k choices in ascending expert id, summed in
    float32 and rounded once to y's dtype."""
    k = idx.shape[1]
    by_expert = torch.sort(idx.long(), dim=1, stable=True).indices          # [N, k] slots
    rows = pos_of.long().view(n_tokens, k).gather(1, by_expert)             # [N, k]
    acc = torch.zeros(n_tokens, y.shape[1], dtype=torch.float32, device=y.device)
    for j in range(k):
        acc = acc + y[rows[:, j]].float()
    return acc.to(y.dtype)


def tile_offsets(counts, block=64):
    tiles = (counts + block - 1) // block
    off = torch.zeros(counts.numel() + 1, dtype=torch.int32, device=counts.device)
    off[1:] = torch.cumsum(tiles, 0)
    return off


def moe_layer(h, router, gate_up, down, top_k, norm_topk_prob):
    idx, w = route(h, router, top_k, norm_topk_prob)
    return experts_loop(h, idx, w, gate_up, down)


# ---------------------------------------------------------------- numpy brute force
def brute_force_layer(h, idx, w, gate_up, down):
    """float64, one (token, slot) at a time, straight from the definition:
    out[t] = sum_s w[t,s] * down[e] @ (silu(gate[e] @ h[t]) * (up[e] @ h[t])), e = idx[t,s]."""
    h, w = np.asarray(h, dtype=np.float64), np.asarray(w, dtype=np.float64)
    gu, dn = np.asarray(gate_up, dtype=np.float64), np.asarray(down, dtype=np.float64)
    idx = np.asarray(idx)
    N, k = idx.shape
    inter = dn.shape[2]
    out = np.zeros_like(h)
    for t in range(N):
        for s in range(k):
            e = int(idx[t, s])
            g = gu[e, :inter] @ h[t]
            u = gu[e, inter:] @ h[t]
            out[t] += w[t, s] * (dn[e] @ (g / (1.0 + np.exp(-g)) * u))
    return out


def brute_force_topk(logits_row, k):
    """Scan for the best remaining (value desc, id asc) candidate k times."""
    v = [float(x) for x in logits_row]
    taken, picks = set(), []
    for _ in range(k):
        best = None
        for e, x in enumerate(v):
            if e in taken:
                continue
            if best is None or x > v[best]:
                best = e
        taken.add(best)
        picks.append(best)
    return picks

"""An OLMoE decoder around the MoE layer: the caller of the hot path.

Counterpart of the reference's switchyard/model.py (the `self.moe(i, h)` hook at :39-42,135)
and of the tensor layout its weights.py defines (:36-69). Attention stays in PyTorch; every
mixture-of-experts layer goes through `moe(layer_index, h[B*T, H]) -> [B*T, H]`, which by
default is `kernels.moe_layer` on the layer's router / gate_up / down tensors.

Built for decode on one GPU: the KV cache is allocated once for the whole generation, rotary
tables are precomputed, and the greedy loop keeps its tokens on the device, so a decode step
is a queue of launches with no host read unless the caller asks for early stopping at `eos`.
On a GPU in fp16 the attention side of a decode step runs on the library's decode kernels
(`step_fused`: eight launches per layer with the MoE layer's, every projection a weight
stream) and a prompt goes through `prefill_fused` (the same row kernels around PyTorch's fused
attention call); fp32 and the CPU use the PyTorch operators (`forward`, `step_static`).
"""

from dataclasses import dataclass

import torch
import torch.nn.functional as F


@dataclass
class Shape:
    vocab: int = 50304
    hidden: int = 2048
    intermediate: int = 1024       # per expert
    layers: int = 16
    heads: int = 16
    kv_heads: int = 16
    head_dim: int = 128
    experts: int = 64
    top_k: int = 8
    norm_topk_prob: bool = False
    rms_eps: float = 1e-5
    rope_theta: float = 10000.0
    clip_qkv: float | None = None

    @classmethod
    def from_hf(cls, c):
        """From a transformers OlmoeConfig (or any object with its attribute names)."""
        heads = c.num_attention_heads
        rope = getattr(c, "rope_parameters", None) or {}
        return cls(vocab=c.vocab_size, hidden=c.hidden_size, intermediate=c.intermediate_size,
                   layers=c.num_hidden_layers, heads=heads, kv_heads=getattr(c, "num_key_value_heads", None) or heads,
                   head_dim=getattr(c, "head_dim", None) or c.hidden_size // heads, experts=c.num_experts,
                   top_k=c.num_experts_per_tok, norm_topk_prob=bool(getattr(c, "norm_topk_prob", False)),
                   rms_eps=getattr(c, "rms_norm_eps", 1e-5),
                   rope_theta=rope.get("rope_theta", getattr(c, "rope_theta", 10000.0)),
                   clip_qkv=getattr(c, "clip_qkv", None))


OLMOE_1B_7B = Shape()


def random_weights(shape, dtype=torch.float16, device="cuda", seed=0, std=0.02):
    """Random-initialised weights in the layout the reference's loader produces: experts stacked
    as gate_up [E, 2I, H] (gate rows first) and down [E, H, I]; norm weights 1."""
    g = torch.Generator(device=device).manual_seed(seed)

    def rnd(*dims):
        return (torch.randn(*dims, generator=g, device=device, dtype=torch.float32) * std).to(dtype)

    s = shape
    qd, kvd = s.heads * s.head_dim, s.kv_heads * s.head_dim
    layers = []
    for _ in range(s.layers):
        layers.append(dict(
            attn_norm=torch.ones(s.hidden, dtype=dtype, device=device),
            wq=rnd(qd, s.hidden), wk=rnd(kvd, s.hidden), wv=rnd(kvd, s.hidden), wo=rnd(s.hidden, qd),
            q_norm=torch.ones(qd, dtype=dtype, device=device), k_norm=torch.ones(kvd, dtype=dtype, device=device),
            mlp_norm=torch.ones(s.hidden, dtype=dtype, device=device),
            router=rnd(s.experts, s.hidden), gate_up=rnd(s.experts, 2 * s.intermediate, s.hidden),
            down=rnd(s.experts, s.hidden, s.intermediate)))
    return dict(embed=rnd(s.vocab, s.hidden), final_norm=torch.ones(s.hidden, dtype=dtype, device=device),
                lm_head=rnd(s.vocab, s.hidden), layers=layers)


def weights_from_hf(state_dict, shape, dtype=None, device=None):
    """The same layout from a transformers OlmoeForCausalLM state dict (stacked or per-expert names)."""
    def get(name):
        t = state_dict[name]
        return t.to(dtype=dtype or t.dtype, device=device or t.device).contiguous()

    layers = []
    for i in range(shape.layers):
        p = f"model.layers.{i}."
        if p + "mlp.experts.gate_up_proj" in state_dict:
            gate_up, down = get(p + "mlp.experts.gate_up_proj"), get(p + "mlp.experts.down_proj")
        else:
            gate_up = torch.stack([torch.cat([get(f"{p}mlp.experts.{e}.gate_proj.weight"),
                                              get(f"{p}mlp.experts.{e}.up_proj.weight")]) for e in range(shape.experts)])
            down = torch.stack([get(f"{p}mlp.experts.{e}.down_proj.weight") for e in range(shape.experts)])
        layers.append(dict(
            attn_norm=get(p + "input_layernorm.weight"), mlp_norm=get(p + "post_attention_layernorm.weight"),
            wq=get(p + "self_attn.q_proj.weight"), wk=get(p + "self_attn.k_proj.weight"),
            wv=get(p + "self_attn.v_proj.weight"), wo=get(p + "self_attn.o_proj.weight"),
            q_norm=get(p + "self_attn.q_norm.weight"), k_norm=get(p + "self_attn.k_norm.weight"),
            router=get(p + "mlp.gate.weight"), gate_up=gate_up, down=down))
    lm_head = get("lm_head.weight") if "lm_head.weight" in state_dict else get("model.embed_tokens.weight")
    return dict(embed=get("model.embed_tokens.weight"), final_norm=get("model.norm.weight"), lm_head=lm_head,
                layers=layers)


def _rms(x, weight, eps):
    # normalise in fp32, cast back, then scale: the order transformers uses
    f = x.float()
    return weight * (f * torch.rsqrt(f.square().mean(-1, keepdim=True) + eps)).to(x.dtype)


def _rotate(x, cos, sin):
    half = x.shape[-1] // 2
    return x * cos + torch.cat([-x[..., half:], x[..., :half]], dim=-1) * sin


class Span:
    """The T positions a forward call appends to a cache (or a whole sequence without one).

    real [B, T]       False where a row holds left padding
    first, end        the cache slots the span occupies
    seen [B]          real tokens of each row before the span
    positions [B, T]  rotary position of each new token: its index among its row's real tokens
    visible           [B, 1, T, end] attention mask: a query sees the slots at or before its own
                      that hold a real token; a padding query, which would see nothing, sees
                      itself (its output is never used, but its softmax must not be empty)."""

    def __init__(self, tokens, cache, real=None):
        B, T = tokens.shape
        dev = tokens.device
        self.real = torch.ones(B, T, dtype=torch.bool, device=dev) if real is None else real
        self.first = cache.filled if cache is not None else 0
        self.end = self.first + T
        self.seen = cache.next_position if cache is not None else torch.zeros(B, dtype=torch.long, device=dev)
        order = self.real.long().cumsum(1)                       # 1-based index among the row's real tokens
        self.positions = (self.seen[:, None] + order - 1).clamp_(min=0)
        if cache is not None:
            cache.real[:, self.first:self.end] = self.real
            slot_real = cache.real[:, :self.end]
        else:
            slot_real = self.real
        query_slot = torch.arange(self.first, self.end, device=dev)[:, None]
        slot = torch.arange(self.end, device=dev)[None, :]
        sees = (slot <= query_slot)[None] & slot_real[:, None, :]
        alone = ~sees.any(-1, keepdim=True)
        self.visible = (sees | (alone & (slot == query_slot)[None]))[:, None]   # broadcast over heads

    def commit(self, cache):
        """The span now belongs to the cache."""
        cache.filled = self.end
        cache.next_position = self.seen + self.real.long().sum(1)


def left_padded(prompts, device):
    """Token lists of unequal length as one right-aligned batch: (tokens [B, P], real [B, P])."""
    lengths = torch.tensor([len(p) for p in prompts])
    width = int(lengths.max())
    real = torch.arange(width)[None, :] >= (width - lengths)[:, None]
    tokens = torch.zeros(len(prompts), width, dtype=torch.long)
    tokens[real] = torch.tensor([t for p in prompts for t in p], dtype=torch.long)   # row by row, in order
    return tokens.to(device), real.to(device)


class KVCache:
    """Keys and values of every layer, [B, kv_heads, capacity, head_dim], allocated once.
    `filled` positions are in use; `real[b, p]` is False where batch row b holds left padding."""

    def __init__(self, shape, batch, capacity, dtype, device):
        dims = (shape.layers, batch, shape.kv_heads, capacity, shape.head_dim)
        self.k = torch.zeros(dims, dtype=dtype, device=device)
        self.v = torch.zeros(dims, dtype=dtype, device=device)
        self.real = torch.zeros(batch, capacity, dtype=torch.bool, device=device)
        self.next_position = torch.zeros(batch, dtype=torch.long, device=device)
        self.filled = 0
        self.capacity = capacity


class Decoder:
    def __init__(self, shape, weights, moe=None, max_positions=4096, attention="auto"):
        """attention: "kernels" (the library's kernels for the decode step and around the prompt's
        attention), "torch" (PyTorch operators throughout), or "auto": kernels where they apply
        (GPU, fp16, head_dim 64 or 128)."""
        self.s, self.w = shape, weights
        self.moe = moe or self.kernel_moe
        self._own_moe = moe is None     # the step may then fold the layer's ends into its neighbours
        dev = weights["embed"].device
        can = (dev.type == "cuda" and weights["embed"].dtype == torch.float16 and shape.head_dim in (64, 128)
               and shape.hidden % 8 == 0 and shape.hidden <= 8192 and shape.heads * shape.head_dim <= 8192)
        if attention == "kernels" and not can:
            raise ValueError("the decode kernels need a GPU, fp16 weights and head_dim 64 or 128")
        self.fused = can if attention == "auto" else attention == "kernels"
        self._wqkv = None
        inv = 1.0 / (shape.rope_theta ** (torch.arange(0, shape.head_dim, 2, device=dev).float() / shape.head_dim))
        ang = torch.outer(torch.arange(max_positions, device=dev).float(), inv)
        table = torch.cat([ang, ang], dim=-1)
        self.cos, self.sin = table.cos().to(weights["embed"].dtype), table.sin().to(weights["embed"].dtype)

    # ---- the hook's default: the gfx950 kernels
    def kernel_moe(self, i, h):
        from . import kernels

        L = self.w["layers"][i]
        return kernels.moe_layer(h, L["router"], L["gate_up"], L["down"], self.s.top_k, self.s.norm_topk_prob)

    # ---- the PyTorch formulation of a forward pass (any device, any dtype)
    def _heads(self, x, weight, norm, n_heads):
        """One of the q / k / v projections of x [B, T, H] as heads [B, n_heads, T, head_dim]."""
        s = self.s
        y = F.linear(x, weight)
        if norm is not None:
            y = _rms(y, norm, s.rms_eps)
        if s.clip_qkv is not None:
            y = y.clamp(-s.clip_qkv, s.clip_qkv)
        return y.unflatten(-1, (n_heads, s.head_dim)).transpose(1, 2)

    def _attend(self, i, x, span, cache):
        """Attention of layer i over the span's new positions (and what the cache already holds)."""
        s, L = self.s, self.w["layers"][i]
        cos, sin = self.cos[span.positions][:, None], self.sin[span.positions][:, None]
        q = _rotate(self._heads(x, L["wq"], L["q_norm"], s.heads), cos, sin)
        k = _rotate(self._heads(x, L["wk"], L["k_norm"], s.kv_heads), cos, sin)
        v = self._heads(x, L["wv"], None, s.kv_heads)
        if cache is not None:
            new = slice(span.first, span.end)
            cache.k[i, :, :, new], cache.v[i, :, :, new] = k, v
            k, v = cache.k[i, :, :, :span.end], cache.v[i, :, :, :span.end]
        a = F.scaled_dot_product_attention(q, k, v, attn_mask=span.visible, enable_gqa=s.kv_heads != s.heads)
        return F.linear(a.transpose(1, 2).flatten(-2), L["wo"])

    @torch.no_grad()
    def forward(self, tokens, cache=None, valid=None):
        """tokens [B, T] -> logits [B, T, vocab]. `valid` [B, T] marks real tokens (False = left
        padding). With a cache the tokens are appended after what it already holds."""
        s, W = self.s, self.w
        B, T = tokens.shape
        span = Span(tokens, cache, valid)
        x = F.embedding(tokens, W["embed"])
        for i in range(s.layers):
            L = W["layers"][i]
            x = x + self._attend(i, _rms(x, L["attn_norm"], s.rms_eps), span, cache)
            h = _rms(x, L["mlp_norm"], s.rms_eps).reshape(B * T, s.hidden)
            x = x + self.moe(i, h).view(B, T, s.hidden)
        if cache is not None:
            span.commit(cache)
        return F.linear(_rms(x, W["final_norm"], s.rms_eps), W["lm_head"])

    @torch.no_grad()
    def prefill_fused(self, tokens, cache, valid=None):
        """`forward` for a prompt on the library's kernels, returning the logits of the last
        position only, [B, vocab]: norms, residual adds, the q/k norm with the rotary embedding
        and the cache write are one launch each over all B*T rows (in PyTorch they are some
        seventy element-wise launches per layer, each a pass over the activations), the three
        input projections are one GEMM, and the lm_head runs on B rows instead of B*T.
        Attention itself is PyTorch's fused scaled-dot-product call under the same mask."""
        from . import kernels

        s, W, E = self.s, self.w, kernels.ext()
        B, T = tokens.shape
        span = Span(tokens, cache, valid)
        wqkv = self._stacked_qkv()
        slot = torch.tensor([span.first], dtype=torch.long, device=tokens.device)
        flat_positions = span.positions.reshape(-1).contiguous()
        x, xn = E.embed_rmsnorm(tokens.reshape(-1).contiguous(), W["embed"], W["layers"][0]["attn_norm"], s.rms_eps)
        for i in range(s.layers):
            L = W["layers"][i]
            after = W["layers"][i + 1]["attn_norm"] if i + 1 < s.layers else W["final_norm"]
            q = E.qk_norm_rope_cache(kernels.dense(xn, wqkv[i]), L["q_norm"], L["k_norm"], s.rms_eps, s.clip_qkv, self.cos,
                                     self.sin, flat_positions, slot, s.heads, s.kv_heads, s.head_dim, cache.k[i], cache.v[i])
            a = F.scaled_dot_product_attention(q.view(B, T, s.heads, s.head_dim).transpose(1, 2),
                                               cache.k[i, :, :, :span.end], cache.v[i, :, :, :span.end],
                                               attn_mask=span.visible, enable_gqa=s.kv_heads != s.heads)
            o = kernels.dense(a.transpose(1, 2).reshape(B * T, s.heads * s.head_dim), L["wo"])
            x, h = E.add_rmsnorm(x, o, L["mlp_norm"], s.rms_eps, x_out=x)
            if self._own_moe and s.top_k <= 64:
                y, pos_of, idx = kernels.experts_rows(h, None, L["gate_up"], L["down"], s.top_k, s.norm_topk_prob,
                                                      router=L["router"])
                x, xn = E.combine_add_rmsnorm(y, pos_of, idx, x, after, s.rms_eps, x_out=x)
            else:
                x, xn = E.add_rmsnorm(x, self.moe(i, h).contiguous(), after, s.rms_eps, x_out=x)
        span.commit(cache)
        return kernels.dense(xn.view(B, T, s.hidden)[:, -1].contiguous(), W["lm_head"])

    def _prefill(self, tokens, cache, valid):
        """Logits of the last prompt position [B, vocab], on the kernels where they apply."""
        if self.fused:
            return self.prefill_fused(tokens, cache, valid)
        return self.forward(tokens, cache, valid)[:, -1]

    # ---- one decode step with every index on the device, so that it can be captured in a HIP graph
    @torch.no_grad()
    def step_static(self, tok, cache, slot, keys):
        """tok [B, 1] -> logits [B, vocab]. `slot` is a one-element device tensor holding the cache
        position to write (the same for every row of a left-padded batch); `keys` is
        arange(capacity). Attention runs over the whole capacity under a mask, shapes never change,
        and nothing depends on a host value: the step is a fixed sequence of launches."""
        s, W = self.s, self.w
        B = tok.shape[0]
        positions = cache.next_position[:, None]
        cache.real.index_fill_(1, slot, True)
        mask = ((keys[None, :] <= slot) & cache.real)[:, None, None, :]
        x = F.embedding(tok, W["embed"])
        for i in range(s.layers):
            L = W["layers"][i]
            xn = _rms(x, L["attn_norm"], s.rms_eps)
            q = _rms(F.linear(xn, L["wq"]), L["q_norm"], s.rms_eps)
            k = _rms(F.linear(xn, L["wk"]), L["k_norm"], s.rms_eps)
            v = F.linear(xn, L["wv"])
            if s.clip_qkv is not None:
                q, k, v = (q.clamp(-s.clip_qkv, s.clip_qkv), k.clamp(-s.clip_qkv, s.clip_qkv),
                           v.clamp(-s.clip_qkv, s.clip_qkv))
            q = q.view(B, 1, s.heads, s.head_dim).transpose(1, 2)
            k = k.view(B, 1, s.kv_heads, s.head_dim).transpose(1, 2)
            v = v.view(B, 1, s.kv_heads, s.head_dim).transpose(1, 2)
            cos, sin = self.cos[positions][:, None], self.sin[positions][:, None]
            q, k = _rotate(q, cos, sin), _rotate(k, cos, sin)
            cache.k[i].index_copy_(2, slot, k)
            cache.v[i].index_copy_(2, slot, v)
            a = F.scaled_dot_product_attention(q, cache.k[i], cache.v[i], attn_mask=mask,
                                               enable_gqa=s.kv_heads != s.heads)
            x = x + F.linear(a.transpose(1, 2).reshape(B, 1, s.heads * s.head_dim), L["wo"])
            h = _rms(x, L["mlp_norm"], s.rms_eps).reshape(B, s.hidden)
            x = x + self.moe(i, h).view(B, 1, s.hidden)
        cache.next_position += 1
        slot += 1
        return F.linear(_rms(x, W["final_norm"], s.rms_eps), W["lm_head"])[:, -1]

    def _stacked_qkv(self):
        """wq, wk, wv of every layer stacked as one [q | k | v] projection, so that the three are
        one weight stream; the dictionary's own entries become views of the stack."""
        if self._wqkv is None:
            self._wqkv = []
            for L in self.w["layers"]:
                stack = torch.cat([L["wq"], L["wk"], L["wv"]]).contiguous()
                qd, kvd = L["wq"].shape[0], L["wk"].shape[0]
                L["wq"], L["wk"], L["wv"] = stack[:qd], stack[qd:qd + kvd], stack[qd + kvd:]
                self._wqkv.append(stack)
        return self._wqkv

    @torch.no_grad()
    def step_fused(self, tok, cache, slot, keys=None, advance=True):
        """The same step as `step_static` on the decode kernels: embedding + RMS norm, the
        stacked q/k/v projection, attention over the cache (with the q/k norm, the rotary
        embedding and the cache write in its prologue), the output projection, residual add +
        RMS norm, and the MoE hook; every projection streams its weights once. With
        advance=False the cache counters are left to the caller (`greedy_advance` moves them
        together with the arg-max)."""
        from . import kernels

        s, W, E = self.s, self.w, kernels.ext()
        wqkv = self._stacked_qkv()
        positions = cache.next_position
        x, xn = E.embed_rmsnorm(tok.reshape(-1), W["embed"], W["layers"][0]["attn_norm"], s.rms_eps)
        for i in range(s.layers):
            L = W["layers"][i]
            after = W["layers"][i + 1]["attn_norm"] if i + 1 < s.layers else W["final_norm"]
            a = E.decode_attention_qkv(kernels.dense(xn, wqkv[i]), L["q_norm"], L["k_norm"], s.rms_eps, s.clip_qkv,
                                       self.cos, self.sin, positions, slot, cache.real, s.heads, s.kv_heads,
                                       s.head_dim, cache.k[i], cache.v[i])
            o = kernels.dense(a, L["wo"])
            if self._own_moe and s.experts <= 1024 and s.top_k <= 64:
                # the router's logits come out of the norm's launch, and combine goes into the next norm's
                if x.shape[0] <= 256 and s.experts <= 128 and s.top_k <= min(8, s.experts):
                    # ... and so do route and sort. On the weight-stream kernels the router weights
                    # are applied where the rows are combined, and the down projection fetches no
                    # scale per row (batch 8: 2.336 -> 2.318 ms per step; on the MFMA tiles of batch
                    # 64 the projection gains nothing and the combine loses 0.5 us)
                    x, h, _, idx, w, counts, offsets, token, wsorted, pos_of = E.add_rmsnorm(
                        x, o, L["mlp_norm"], s.rms_eps, x_out=x, router=L["router"], front=(s.top_k, s.norm_topk_prob))
                    mode = kernels._auto(x.shape[0], idx.numel(), s.experts)
                    if mode == "gemv":
                        wsorted = None
                    else:
                        w = None
                    y = kernels.ffn(h, token, offsets, counts, wsorted, L["gate_up"], L["down"], idx.numel(), mode)
                else:
                    x, h, logits = E.add_rmsnorm(x, o, L["mlp_norm"], s.rms_eps, x_out=x, router=L["router"])
                    y, pos_of, idx = kernels.experts_rows(h, logits, L["gate_up"], L["down"], s.top_k, s.norm_topk_prob)
                    w = None
                x, xn = E.combine_add_rmsnorm(y, pos_of, idx, x, after, s.rms_eps, x_out=x, w=w)
            else:
                x, h = E.add_rmsnorm(x, o, L["mlp_norm"], s.rms_eps, x_out=x)
                x, xn = E.add_rmsnorm(x, self.moe(i, h), after, s.rms_eps, x_out=x)
        if advance:
            cache.next_position += 1
            slot += 1
        return kernels.dense(xn, W["lm_head"])

    def step(self, tok, cache, slot, keys):
        """One decode step for every sequence: tok [B, 1] -> logits [B, vocab]; advances the cache."""
        return self.step_fused(tok, cache, slot) if self.fused else self.step_static(tok, cache, slot, keys)

    @torch.no_grad()
    def generate_graph(self, prompts, max_new_tokens, return_first_logits=False, timings=None):
        """Greedy decoding with the decode step captured once in a HIP graph and replayed per
        token: prefill eagerly, then one graph launch per generated token and no host work in
        between (no early stop at an eos token). Same tokens as `generate`. If `timings` is a
        dict, the wall times of the prefill and of the replay loop are stored in it (this adds two
        device synchronisations)."""
        import time
        dev, dtype = self.w["embed"].device, self.w["embed"].dtype
        tokens, valid = left_padded(prompts, dev)
        B, P = tokens.shape
        cache = KVCache(self.s, B, P + max_new_tokens, dtype, dev)
        if timings is not None:
            torch.cuda.synchronize()
            t0 = time.perf_counter()
        first_logits = self._prefill(tokens, cache, valid)
        if timings is not None:
            torch.cuda.synchronize()
            timings["prefill_s"] = time.perf_counter() - t0
        out = torch.zeros(B, max_new_tokens, dtype=torch.long, device=dev)
        tok = first_logits.argmax(-1)[:, None].clone()
        out[:, 0] = tok[:, 0]
        if max_new_tokens > 1:
            slot = torch.tensor([cache.filled], dtype=torch.long, device=dev)
            col = torch.ones(1, dtype=torch.long, device=dev)       # column of `out` the next token goes to
            keys = torch.arange(cache.capacity, device=dev)

            if self.fused:
                from . import kernels
                base = cache.next_position - 1          # column 1 of `out` is due now

                def one_token():
                    logits = self.step_fused(tok, cache, slot, advance=False)
                    kernels.ext().greedy_advance(logits, tok, out, base, cache.next_position, slot)
            else:
                def one_token():
                    logits = self.step_static(tok, cache, slot, keys)
                    tok.copy_(logits.argmax(-1)[:, None])
                    out.index_copy_(1, col, tok)
                    col.add_(1)

            # warm up on a side stream (allocator, kernel loading), then restore the state it touched
            saved = (cache.next_position.clone(), slot.clone(), col.clone(), tok.clone(), cache.real.clone(), out.clone())
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                one_token()
            torch.cuda.current_stream().wait_stream(side)
            cache.next_position.copy_(saved[0]); slot.copy_(saved[1]); col.copy_(saved[2]); tok.copy_(saved[3])
            cache.real.copy_(saved[4]); out.copy_(saved[5])
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                one_token()
            cache.next_position.copy_(saved[0]); slot.copy_(saved[1]); col.copy_(saved[2]); tok.copy_(saved[3])
            cache.real.copy_(saved[4]); out.copy_(saved[5])
            if timings is not None:
                torch.cuda.synchronize()
                t0 = time.perf_counter()
            for _ in range(max_new_tokens - 1):
                graph.replay()
            if timings is not None:
                torch.cuda.synchronize()
                timings["decode_s"] = time.perf_counter() - t0
                timings["decode_steps"] = max_new_tokens - 1
        rows = out.tolist()
        return (rows, first_logits) if return_first_logits else rows

    @torch.no_grad()
    def generate(self, prompts, max_new_tokens, eos=None, return_first_logits=False):
        """Greedy decoding of a batch of token lists, left-padded internally. Returns the generated
        tokens of each prompt (cut after `eos` if given). Without `eos` nothing is read back from
        the device until the end."""
        dev, dtype = self.w["embed"].device, self.w["embed"].dtype
        tokens, valid = left_padded(prompts, dev)
        B, P = tokens.shape
        cache = KVCache(self.s, B, P + max_new_tokens, dtype, dev)
        logits = self._prefill(tokens, cache, valid)
        first_logits = logits
        out = torch.zeros(B, max_new_tokens, dtype=torch.long, device=dev)
        steps = 0
        alive = torch.ones(B, dtype=torch.bool, device=dev)
        if self.fused:
            # the launches `generate_graph` replays, issued one by one: the step on the decode
            # kernels, then arg-max, append and counters in one launch
            from . import kernels
            tok = logits.argmax(-1)[:, None].clone()
            out[:, 0] = tok[:, 0]
            steps = 1
            slot = torch.tensor([cache.filled], dtype=torch.long, device=dev)
            base = cache.next_position - 1
            for step in range(1, max_new_tokens):
                if eos is not None:
                    alive &= tok[:, 0] != eos
                    if not bool(alive.any()):
                        break
                step_logits = self.step_fused(tok, cache, slot, advance=False)
                kernels.ext().greedy_advance(step_logits, tok, out, base, cache.next_position, slot)
                cache.filled += 1
                steps = step + 1
        else:
            for step in range(max_new_tokens):
                nxt = logits.argmax(-1)
                out[:, step] = nxt
                steps = step + 1
                if eos is not None:
                    alive &= nxt != eos
                    if not bool(alive.any()):
                        break
                if step + 1 < max_new_tokens:
                    logits = self.forward(nxt[:, None], cache)[:, -1]
        rows = out[:, :steps].tolist()
        if eos is not None:
            rows = [r[:r.index(eos) + 1] if eos in r else r for r in rows]
        return (rows, first_logits) if return_first_logits else rows

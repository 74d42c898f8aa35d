"""Parity of the HIP kernels with the CPU oracle, through the C ABI. Needs an MI355X.

Integer outputs (expert ids, counts, offsets, sorted order, pos_of) and pure permutations
(wsorted) are compared bit for bit. Floating-point outputs use the reference's own criterion
(tests/test_kernels_cuda.py:48-53): error against the fp32 loop at most twice the fp16 loop's,
floor 2e-3; and max abs error <= 2e-2 against the fp16 per-expert loop."""

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import cases
from oracle import c_oracle
from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu

DEV = "cuda"
FP16_TOL = 2e-2     # max abs error against the fp16 per-expert loop
WEIGHT_TOL = 1e-3   # router weights (fp32 sum order differs from the library softmax)


@pytest.fixture(scope="module")
def K():
    from switchyard_amd import kernels

    return kernels


@pytest.fixture(scope="module")
def olmoe():
    """Router and expert weights of one OLMoE-1B-7B layer (64 experts, 2048 -> 1024 -> 2048)."""
    _, router, gu, dn = cases.layer(1)
    return router.to(DEV), gu.to(DEV), dn.to(DEV)


def hidden(N, H=2048, seed=0):
    return torch.randn(N, H, generator=torch.Generator().manual_seed(seed + 1000 + N)).half().to(DEV)


def check_route(K, logits, k, norm):
    idx, w = K.ext().route(logits, k, norm)
    oidx, ow = O.route_logits(logits.cpu(), k, norm)
    assert idx.dtype == torch.int32 and w.dtype == logits.dtype
    assert torch.equal(idx.cpu().long(), oidx), "expert ids differ from the oracle"
    assert (w.cpu().float() - ow.float()).abs().max().item() < WEIGHT_TOL
    return idx, w


# ------------------------------------------------------------------ route
@pytest.mark.parametrize("E,k", [(8, 2), (64, 8), (60, 4), (128, 8), (16, 4), (100, 1), (3, 3)])
@pytest.mark.parametrize("norm", [False, True])
def test_route_ids_are_bit_exact(K, E, k, norm):
    h, router, _, _ = cases.unit_layer(300, E=E, k=k)
    logits = F.linear(h.to(DEV), router.to(DEV)).contiguous()
    idx, w = check_route(K, logits, k, norm)
    cidx, _ = c_oracle.route(logits.float().cpu().numpy(), k, norm)
    assert np.array_equal(idx.cpu().numpy(), cidx)
    # the reference's own criterion: the same experts as softmax -> topk on almost every row
    ridx = torch.topk(torch.softmax(logits.float(), -1), k, dim=-1).indices
    same = (idx.long().sort(-1).values == ridx.sort(-1).values).all(-1)
    assert same.float().mean().item() > 0.99


@pytest.mark.parametrize("N", [1, 8, 4096])
def test_route_on_the_benchmark_layer_with_ties(K, olmoe, N):
    router = olmoe[0]
    logits = F.linear(hidden(N), router).contiguous()
    check_route(K, logits, 8, False)
    if N == 4096:
        srt = torch.sort(logits.float(), dim=-1, descending=True).values
        assert int((srt[:, 7] == srt[:, 8]).sum()) > 0, "expected ties across the top-8 edge"


def test_route_all_equal_logits_picks_the_lowest_ids(K):
    logits = torch.zeros(5, 64, dtype=torch.float16, device=DEV)
    idx, w = K.ext().route(logits, 8, False)
    assert idx.cpu().tolist() == [list(range(8))] * 5
    assert torch.allclose(w.float().cpu(), torch.full((5, 8), 1 / 64), atol=1e-4)
    idx, w = K.ext().route(logits, 8, True)
    assert torch.allclose(w.float().cpu(), torch.full((5, 8), 1 / 8), atol=1e-3)


def test_route_fp32_logits_config1(K):
    h, router, _, _ = cases.layer(32, E=16, k=4, H=128, I=64, dtype=torch.float32)
    logits = F.linear(h, router).to(DEV).contiguous()
    idx, w = check_route(K, logits, 4, False)
    assert w.dtype == torch.float32


def test_route_rejects_what_the_reference_rejects(K):
    with pytest.raises(RuntimeError):
        K.ext().route(torch.zeros(4, 200, dtype=torch.float16, device=DEV), 8, False)
    with pytest.raises(RuntimeError):
        K.ext().route(torch.zeros(4, 64, dtype=torch.float16, device=DEV), 9, False)
    idx, w = K.ext().route(torch.zeros(0, 64, dtype=torch.float16, device=DEV), 8, False)
    assert idx.shape == (0, 8) and w.shape == (0, 8)


# ------------------------------------------------------------------ sort
def check_sort(K, idx, w, E):
    a = K.ext().sort_by_expert(idx, w, E)
    b = K.ext().sort_by_expert(idx, w, E)
    assert all(torch.equal(x, y) for x, y in zip(a, b)), "two runs differ"
    counts, offsets, token, wsorted, pos_of = (t.cpu() for t in a)
    p = O.plan(idx.cpu().long(), w.cpu(), E)
    assert torch.equal(counts.long(), p.counts)
    assert torch.equal(offsets.long(), p.offsets)
    assert torch.equal(token.long(), p.token)
    assert torch.equal(pos_of.long(), p.pos_of)
    assert torch.equal(wsorted.view(torch.int16), p.weight.view(torch.int16))
    return a


@pytest.mark.parametrize("N,E,k", [(1, 64, 8), (7, 64, 8), (64, 64, 8), (333, 64, 8), (999, 64, 8), (1024, 64, 8),
                                   (1025, 64, 8), (4096, 64, 8), (40000, 64, 8), (300, 60, 4), (300, 128, 8),
                                   (50, 8, 2), (5, 200, 3), (3000, 512, 8), (32, 16, 4)])
def test_sort_is_bit_exact_stable_and_deterministic(K, N, E, k):
    g = torch.Generator().manual_seed(N + E)
    logits = torch.randn(N, E, generator=g)
    idx = torch.topk(logits, k, dim=-1).indices.int().to(DEV)
    w = torch.rand(N, k, generator=g).half().to(DEV)
    check_sort(K, idx, w, E)


def test_sort_known_answer_from_the_reference_tests(K):
    g = cases.golden_sort_vector()
    idx = torch.tensor(g["idx"], dtype=torch.int32, device=DEV)
    w = torch.tensor(g["w"], dtype=torch.float16, device=DEV)
    counts, offsets, token, wsorted, pos_of = K.ext().sort_by_expert(idx, w, g["n_experts"])
    assert counts.tolist() == g["counts"] and offsets.tolist() == g["offsets"]
    assert token.tolist() == g["token"] and pos_of.tolist() == g["pos_of"]
    assert torch.allclose(wsorted.float().cpu(), torch.tensor(g["weight"]), atol=1e-3)


def test_sort_with_repeats_skew_and_fp32_weights(K):
    g = torch.Generator().manual_seed(5)
    idx = torch.randint(0, 4, (5000, 8), generator=g).int().to(DEV)      # heavy repeats inside a token
    w = torch.rand(5000, 8, generator=g).to(DEV)                          # fp32 weights
    a = K.ext().sort_by_expert(idx, w, 64)
    p = O.plan(idx.cpu().long(), w.cpu(), 64)
    assert torch.equal(a[2].cpu().long(), p.token) and torch.equal(a[4].cpu().long(), p.pos_of)
    assert torch.equal(a[3].cpu(), p.weight)
    same = torch.zeros(777, 8, dtype=torch.int32, device=DEV) + 63         # every choice the same expert
    check_sort(K, same, torch.rand(777, 8).half().to(DEV), 64)


def test_sort_of_nothing(K):
    idx = torch.zeros(0, 8, dtype=torch.int32, device=DEV)
    w = torch.zeros(0, 8, dtype=torch.float16, device=DEV)
    counts, offsets, token, wsorted, pos_of = K.ext().sort_by_expert(idx, w, 64)
    assert counts.tolist() == [0] * 64 and offsets.tolist() == [0] * 65 and token.numel() == 0


# ------------------------------------------------------------------ combine
@pytest.mark.parametrize("N,k,H", [(1, 8, 2048), (33, 8, 256), (500, 4, 128), (64, 1, 64), (20, 3, 2056)])
def test_combine_is_bit_exact(K, N, k, H):
    g = torch.Generator().manual_seed(N)
    E = 64
    idx = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(N)]).int()
    p = O.plan(idx.long(), torch.zeros(N, k), E)
    y = torch.randn(N * k, H, generator=g).half()
    want = O.combine_rows(y, p.pos_of, idx, N)
    got = K.ext().combine(y.to(DEV), p.pos_of.int().to(DEV), idx.to(DEV), N)
    assert torch.equal(got.cpu().view(torch.int16), want.view(torch.int16))


# ------------------------------------------------------------------ the grouped projections
def fp16_graph(x, token, offsets, wsorted, gu, dn):
    return O.ffn_rows(x, token, offsets, wsorted, gu, dn)


@pytest.mark.parametrize("mode", ["gemv", "gemm"])
@pytest.mark.parametrize("N,H,I,E,k", [(1, 256, 128, 64, 8), (7, 256, 128, 64, 8), (64, 256, 128, 64, 8),
                                       (333, 256, 128, 64, 8), (40, 128, 64, 16, 4), (100, 96, 40, 8, 2),
                                       (50, 2048, 1024, 8, 2), (300, 512, 72, 5, 3)])
def test_ffn_rows_match_the_fp16_graph(K, mode, N, H, I, E, k):
    if mode == "gemm" and (H % 32 or I % 32):
        pytest.skip("the MFMA tile kernel needs K % 32 == 0, as the reference's does")
    h, router, gu, dn = (t.to(DEV) for t in cases.unit_layer(N, E=E, k=k, H=H, I=I))
    idx, w = K.route(h, router, k, False)
    counts, offsets, token, wsorted, pos_of = K.ext().sort_by_expert(idx, w, E)
    y = K.ffn(h, token, offsets, counts, wsorted, gu, dn, N * k, mode)
    want16 = fp16_graph(h, token, offsets, wsorted, gu, dn)
    want32 = fp16_graph(h.float(), token, offsets, wsorted.float(), gu.float(), dn.float())
    err, err16 = (y.float() - want32).abs().max().item(), (want16.float() - want32).abs().max().item()
    assert err <= max(2 * err16, 2e-3), (err, err16)
    assert (y.float() - want16.float()).abs().max().item() <= FP16_TOL


@pytest.mark.parametrize("swiglu", [True, False])
@pytest.mark.parametrize("fn", ["grouped_gemv", "grouped_gemm"])
def test_grouped_kernels_plain_and_ragged_columns(K, fn, swiglu):
    # Nout not a multiple of the tile / group width, no gather, no scale: the <0,0> variant too
    E, K_, Nout, rows = 6, 64, 44, 150
    g = torch.Generator().manual_seed(9)
    A = torch.randn(rows, K_, generator=g).half().to(DEV)
    B = (torch.randn(E, Nout * (2 if swiglu else 1), K_, generator=g) * K_ ** -0.5).half().to(DEV)
    counts = torch.tensor([0, 17, 1, 100, 0, 32])
    offsets = torch.zeros(E + 1, dtype=torch.int32)
    offsets[1:] = torch.cumsum(counts, 0)
    call = getattr(K.ext(), fn)
    args = (A, None, B, offsets.to(DEV)) + ((None, 0) if fn == "grouped_gemm" else ()) + (rows, swiglu, None)
    got = call(*args).float().cpu()
    want = torch.empty(rows, Nout)
    for e in range(E):
        s, t = int(offsets[e]), int(offsets[e + 1])
        r = F.linear(A[s:t].float(), B[e].float()).cpu()
        # the kernels' rounding points (moe_kernels.cu:253-259,373-378): gate, up, silu(gate) and the
        # product are each rounded to f16; the plain projection rounds its fp32 sum once
        want[s:t] = F.silu(r[:, :Nout].half().float()).half().float() * r[:, Nout:].half().float() if swiglu \
            else r.half().float()
    assert got.shape == (rows, Nout)
    # one rounding to f16 of differently ordered fp32 sums: half-precision ulps, and a floor of one
    # ulp at 1 for outputs near zero
    assert torch.allclose(got, want, rtol=2.0 ** -9, atol=1e-3)


@pytest.mark.parametrize("swiglu", [True, False])
def test_grouped_gemv_with_many_experts(K, swiglu):
    """150 experts with 0 to 5 rows each: the list of used experts spans several 64-lane scans."""
    E, K_, Nout = 150, 256, 24
    counts = torch.tensor([(3 * i) % 6 for i in range(E)])
    rows = int(counts.sum())
    g = torch.Generator().manual_seed(3)
    src = torch.randn(40, K_, generator=g).half()
    a_rows = torch.randint(0, 40, (rows,), generator=g).int()
    B = (torch.randn(E, Nout * (2 if swiglu else 1), K_, generator=g) * K_ ** -0.5).half()
    scale = None if swiglu else torch.rand(rows, generator=g).half()
    offsets = torch.zeros(E + 1, dtype=torch.int32)
    offsets[1:] = torch.cumsum(counts, 0)
    got = K.ext().grouped_gemv(src.to(DEV), a_rows.to(DEV), B.to(DEV), offsets.to(DEV), rows, swiglu,
                               None if scale is None else scale.to(DEV)).float().cpu()
    A = src[a_rows.long()]
    want = torch.empty(rows, Nout)
    for e in range(E):
        s, t = int(offsets[e]), int(offsets[e + 1])
        r = F.linear(A[s:t].float(), B[e].float())
        want[s:t] = F.silu(r[:, :Nout].half().float()).half().float() * r[:, Nout:].half().float() if swiglu \
            else r.half().float() * scale[s:t, None].float()
    assert (got - want).abs().max().item() < 1e-2


@pytest.mark.parametrize("swiglu", [True, False])
@pytest.mark.parametrize("counts,K_,Nout", [
    ([40, 0, 64, 1, 33, 90], 64, 72),               # about 38 rows per expert: the 64-row tile
    ([100, 128, 0, 97, 60, 129], 96, 200),          # about 86: the 128-row tile
    ([300, 0, 257, 1, 512, 130, 256, 31], 64, 72),  # about 186: the 256-row tile, one K slice
    ([300, 0, 257, 1, 512, 130, 256, 31], 128, 300),     # two K slices, fewer than the loads in flight
    ([300, 0, 257, 1, 512, 130, 256, 31], 448, 256),     # seven slices
    ([300, 0, 257, 1, 512, 130, 256, 31], 96, 128),      # K % 64 != 0: falls back to the 128-row tile
    ([1500, 2, 700], 192, 136),                     # many row tiles per expert, ragged columns
    ([(7 * i) % 23 for i in range(150)], 64, 40),         # 150 experts (several 64-lane scans), about 11 rows each
    ([((11 * i) % 7) * 90 for i in range(130)], 128, 264),   # 130 experts, 0 to 540 rows: the 256-row tile
    # the 256-row tile as one stream per compute unit (four or more K slices, at most 128 experts):
    ([300 + (i % 5) * 40 for i in range(100)], 256, 204),    # two experts per lane of the tile table; columns a multiple of 4 only
    ([256] * 8, 256, 256),                                   # fewer tiles than workgroups, all of them full
    ([5000, 3000, 1, 0, 257], 320, 201),                     # five slices, odd column count, 52 tiles of one expert
    ([513, 576, 577, 129, 160, 161, 31, 32, 33, 700], 512, 136),   # every tile height from 1 to 8 blocks
])
def test_grouped_gemm_every_tile_kind(K, counts, K_, Nout, swiglu):
    """Gathered rows, per-row scale (plain projection) or SwiGLU, experts with 0, 1 and many rows:
    grouped_gemm picks its tile from the mean rows per expert, so the shapes walk through all
    three tile kinds and the short-K corners of the one that keeps several slices in flight."""
    E, rows = len(counts), sum(counts)
    g = torch.Generator().manual_seed(rows + K_)
    src = torch.randn(rows // 2 + 3, K_, generator=g).half()
    a_rows = torch.randint(0, src.shape[0], (rows,), generator=g).int()
    B = (torch.randn(E, Nout * (2 if swiglu else 1), K_, generator=g) * K_ ** -0.5).half()
    scale = None if swiglu else torch.rand(rows, generator=g).half()
    offsets = torch.zeros(E + 1, dtype=torch.int32)
    offsets[1:] = torch.cumsum(torch.tensor(counts), 0)
    got = K.ext().grouped_gemm(src.to(DEV), a_rows.to(DEV), B.to(DEV), offsets.to(DEV), None, 0, rows, swiglu,
                               None if scale is None else scale.to(DEV)).float().cpu()
    A = src[a_rows.long()]
    want = torch.empty(rows, Nout)
    for e in range(E):
        s, t = int(offsets[e]), int(offsets[e + 1])
        r = F.linear(A[s:t].float(), B[e].float())
        want[s:t] = F.silu(r[:, :Nout].half().float()).half().float() * r[:, Nout:].half().float() if swiglu \
            else r.half().float() * scale[s:t, None].float()
    assert got.shape == (rows, Nout)
    # one rounding to f16 of differently ordered fp32 sums: an absolute floor plus half-precision ulps
    assert torch.allclose(got, want, rtol=2.0 ** -9, atol=1e-2)


def test_grouped_gemm_stream_tile_with_operands_at_odd_addresses(K):
    """The 256-row tile reads row numbers and scales in runs through the scalar cache, from the
    4-byte word at or below where they start and moved up where a run would pass the end: the
    scales start 2 bytes and the row numbers 4 bytes into their allocations here, and the last
    expert ends the list with a block of a single row."""
    counts, K_, Nout = [300, 417, 1, 290, 513], 256, 256
    E, rows = len(counts), sum(counts)
    g = torch.Generator().manual_seed(5)
    src = torch.randn(400, K_, generator=g).half()
    a_rows = torch.randint(0, 400, (rows,), generator=g).int()
    B = (torch.randn(E, Nout, K_, generator=g) * K_ ** -0.5).half()
    scale = torch.rand(rows, generator=g).half()
    offsets = torch.zeros(E + 1, dtype=torch.int32)
    offsets[1:] = torch.cumsum(torch.tensor(counts), 0)
    scale_dev = torch.cat([torch.zeros(1, dtype=torch.float16), scale]).to(DEV)[1:]
    rows_dev = torch.cat([torch.zeros(1, dtype=torch.int32), a_rows]).to(DEV)[1:]
    assert scale_dev.data_ptr() % 4 == 2 and rows_dev.data_ptr() % 8 == 4
    got = K.ext().grouped_gemm(src.to(DEV), rows_dev, B.to(DEV), offsets.to(DEV), None, 0, rows, False, scale_dev).float().cpu()
    A = src[a_rows.long()]
    want = torch.empty(rows, Nout)
    for e in range(E):
        s, t = int(offsets[e]), int(offsets[e + 1])
        want[s:t] = F.linear(A[s:t].float(), B[e].float()).half().float() * scale[s:t, None].float()
    assert torch.allclose(got, want, rtol=2.0 ** -9, atol=1e-2)


# ------------------------------------------------------------------ the layer, the reference's test
@pytest.mark.parametrize("N", [1, 7, 64, 333, 2048])
@pytest.mark.parametrize("skew", [0.0, 2.0])
@pytest.mark.parametrize("mode", ["gemv", "gemm", "auto"])
def test_moe_layer_matches_the_reference_loop(K, N, skew, mode):
    h, router, gu, dn = (t.to(DEV) for t in cases.unit_layer(N, skew=skew))
    ridx, rw = O.route(h, router, 8, False)
    want = O.experts_loop(h.float(), ridx, rw.float(), gu.float(), dn.float())       # fp32 loop
    half = O.experts_loop(h, ridx, rw, gu, dn).float()                               # fp16 loop
    got = K.experts(h, ridx.int(), rw, gu, dn, mode).float()
    err, err_half = (got - want).abs().max().item(), (half - want).abs().max().item()
    assert err <= max(2 * err_half, 2e-3), (err, err_half)
    assert (got - half).abs().max().item() <= FP16_TOL


def test_empty_experts_a_single_token_and_no_tokens(K):
    h, router, gu, dn = (t.to(DEV) for t in cases.unit_layer(1))
    out = K.moe_layer(h, router, gu, dn, 8, False)
    ridx, rw = O.route(h, router, 8, False)
    want = O.experts_loop(h.float(), ridx, rw.float(), gu.float(), dn.float())
    assert (out.float() - want).abs().max().item() < 2e-3
    none = K.moe_layer(h[:0], router, gu, dn, 8, False)
    assert none.shape == (0, 256)


def test_config1_tiny_layer(K):
    # hidden 128, intermediate 64, 16 experts, top-4, 32 tokens: oracle in fp32 on the CPU,
    # kernels on the same values in fp16; ids and order are compared on identical fp32 logits
    h, router, gu, dn = cases.layer(32, E=16, k=4, H=128, I=64, dtype=torch.float32)
    logits = F.linear(h, router)
    oidx, ow = O.route_logits(logits, 4, False)
    idx, w = K.ext().route(logits.to(DEV), 4, False)
    assert torch.equal(idx.cpu().long(), oidx)
    check_sort(K, idx, w, 16)
    want = O.experts_loop(h, oidx, ow, gu, dn)
    for mode in ("gemv", "gemm"):
        got = K.experts(h.half().to(DEV), idx, w.half(), gu.half().to(DEV), dn.half().to(DEV), mode)
        assert (got.float().cpu() - want).abs().max().item() < 2e-3


# ------------------------------------------------------------------ the benchmark layer at full size
def loop_on_gpu(h, router, gu, dn):
    idx, w = O.route(h, router, 8, False)
    return idx, w, O.experts_loop(h, idx, w, gu, dn)


@pytest.mark.parametrize("N,mode", [(1, "gemv"), (8, "gemv"), (16, "gemv"), (32, "gemv"), (32, "auto"),
                                    (256, "gemm"), (1024, "gemm"), (4096, "gemm"), (4096, "auto"), (256, "gemv")])
def test_olmoe_layer_decode_and_prefill(K, olmoe, N, mode):
    router, gu, dn = olmoe
    h = hidden(N)
    got = K.moe_layer(h, router, gu, dn, 8, False, mode)
    idx, w, half = loop_on_gpu(h, router, gu, dn)
    kidx, kw = K.route(h, router, 8, False)
    assert torch.equal(kidx.long(), idx)
    err16 = (got.float() - half.float()).abs().max().item()
    assert err16 <= FP16_TOL
    if N <= 256:
        want = O.experts_loop(h.float(), idx, w.float(), gu.float(), dn.float())
        err, err_half = (got.float() - want).abs().max().item(), (half.float() - want).abs().max().item()
        assert err <= max(2 * err_half, 2e-3), (err, err_half)


@pytest.mark.parametrize("N", [17, 24, 32, 64, 1024])   # 17-32: "auto" decides from the mean and may meet > 16 rows in an expert
@pytest.mark.parametrize("kind", ["zipf", "adversarial"])
def test_skewed_routing_is_exact_and_deterministic(K, olmoe, N, kind):
    router, gu, dn = olmoe
    h = hidden(N)
    bias = (cases.zipf_bias(alpha=1.0) if kind == "zipf" else cases.adversarial_bias()).to(DEV)
    logits = (F.linear(h, router).float() + bias).half().contiguous()
    idx, w = check_route(K, logits, 8, False)
    counts = check_sort(K, idx, w, 64)[0]
    if kind == "adversarial":
        assert counts.tolist() == [N] * 8 + [0] * 56
    else:
        assert counts.max().item() >= (3 if N >= 64 else 2.5) * counts.float().mean().item()
    half = O.experts_loop(h, idx.long(), w, gu, dn)
    for mode in ("gemv", "gemm", "auto"):
        a = K.experts(h, idx, w, gu, dn, mode)
        b = K.experts(h, idx, w, gu, dn, mode)
        assert torch.equal(a, b), "two runs differ"
        assert (a.float() - half.float()).abs().max().item() <= FP16_TOL


def test_every_token_on_the_same_eight_experts_at_4096_tokens(K, olmoe):
    """The most lopsided tile list the MFMA stream can see, through moe_layer: a constant feature
    in h and a router that weighs it send all 4096 tokens to experts 0..7, so eight experts have
    4096 rows (16 row tiles each) and 56 have none."""
    router, gu, dn = olmoe
    N = 4096
    h = hidden(N).clone()
    h[:, 0] = 1.0
    router = router.clone()
    router[:, 0] = 0.0
    router[:8, 0] = 100.0
    idx, w = K.route(h, router, 8, False)
    assert torch.bincount(idx.flatten().long(), minlength=64).tolist() == [N] * 8 + [0] * 56
    a = K.moe_layer(h, router, gu, dn, 8, False)
    b = K.moe_layer(h, router, gu, dn, 8, False)
    assert torch.equal(a, b), "two runs differ"
    half = O.experts_loop(h, idx.long(), w, gu, dn)
    assert (a.float() - half.float()).abs().max().item() <= FP16_TOL
    assert torch.equal(K.experts(h, idx, w, gu, dn, "gemm"), a)


@pytest.mark.parametrize("N,mode", [(32, "gemv"), (4096, "gemm")])
def test_full_size_properties(K, olmoe, N, mode):
    """Size-independent checks at the benchmark's sizes: a permutation of the tokens permutes
    the output bit for bit, doubling the router weights doubles it (exactly, except where an
    f16 intermediate is subnormal), and the two kernels agree."""
    router, gu, dn = olmoe
    h = hidden(N)
    idx, w = K.route(h, router, 8, False)
    out = K.experts(h, idx, w, gu, dn, mode)
    perm = torch.randperm(N, generator=torch.Generator().manual_seed(1)).to(DEV)
    same = torch.equal(K.experts(h[perm], idx[perm], w[perm], gu, dn, mode), out[perm])
    assert same, "a permutation of the tokens changed some output bits"
    doubled = K.experts(h, idx, w * 2, gu, dn, mode)
    # subnormal f16 rows shift the fp32 sum by < 1e-6, which can move the final rounding by one ulp
    assert torch.allclose(doubled.float(), 2 * out.float(), rtol=2.0 ** -10, atol=2.0 ** -23)
    other = K.experts(h, idx, w, gu, dn, "gemm" if mode == "gemv" else "gemv")
    assert (other.float() - out.float()).abs().max().item() < 2e-3


# ------------------------------------------------------------------ route + sort in one launch (decode)
@pytest.mark.parametrize("N,E,k,H", [(1, 64, 8, 2048), (8, 64, 8, 2048), (33, 64, 8, 2048), (64, 64, 8, 256),
                                     (256, 64, 8, 256), (7, 128, 8, 512), (20, 16, 4, 128), (5, 60, 3, 64),
                                     (20, 16, 3, 128), (64, 64, 1, 256)])   # more tokens than wavefronts, one-wavefront sort
@pytest.mark.parametrize("norm", [False, True])
def test_route_sort_in_one_launch(K, N, E, k, H, norm):
    """Bit for bit what route followed by sort_by_expert gives, and what the oracle gives."""
    g = torch.Generator().manual_seed(N * 7 + E)
    h = torch.randn(N, H, generator=g).half().to(DEV)
    router = (torch.randn(E, H, generator=g) * H ** -0.5).half().to(DEV)
    logits = F.linear(h, router).contiguous()
    idx, w, counts, offsets, token, wsorted, pos_of = K.ext().route_sort(logits, k, norm)
    ridx, rw = K.ext().route(logits, k, norm)
    assert torch.equal(idx, ridx) and torch.equal(w, rw)
    for a, b in zip((counts, offsets, token, wsorted, pos_of), K.ext().sort_by_expert(ridx, rw, E)):
        assert torch.equal(a, b)
    oidx, ow = O.route_logits(logits.cpu(), k, norm)
    assert torch.equal(idx.cpu().long(), oidx)
    assert (w.cpu().float() - ow.float()).abs().max().item() < WEIGHT_TOL
    p = O.plan(oidx, w.cpu(), E)
    assert torch.equal(counts.cpu().long(), p.counts) and torch.equal(offsets.cpu().long(), p.offsets)
    assert torch.equal(token.cpu().long(), p.token) and torch.equal(pos_of.cpu().long(), p.pos_of)
    assert torch.equal(wsorted.cpu().view(torch.int16), p.weight.view(torch.int16))


@pytest.mark.parametrize("N,E,k,H", [(1, 64, 8, 2048), (8, 64, 8, 2048), (9, 64, 8, 2048), (16, 64, 8, 2048),
                                     (64, 64, 8, 2048), (256, 64, 8, 256), (7, 128, 8, 512), (20, 16, 3, 128),
                                     (5, 60, 3, 64), (64, 64, 1, 256), (33, 100, 5, 1024),
                                     (256, 128, 8, 8192), (12, 64, 8, 2056)])   # the largest shape; a ragged row
@pytest.mark.parametrize("norm", [False, True])
def test_router_logits_route_and_sort_in_one_launch(K, N, E, k, H, norm):
    """Bit for bit what router_logits, route and sort_by_expert give in three launches, and the
    oracle's route and plan on those logits; called three times in a row, because every launch
    must leave its counter as it found it."""
    g = torch.Generator().manual_seed(N * 11 + E)
    h = torch.randn(N, H, generator=g).half().to(DEV)
    router = (torch.randn(E, H, generator=g) * H ** -0.5).half().to(DEV)
    ext = K.ext()
    rlogits = ext.router_logits(h, router)
    ridx, rw = ext.route(rlogits, k, norm)
    rsort = ext.sort_by_expert(ridx, rw, E)
    for _ in range(3):
        logits, idx, w, *sort = ext.router_route_sort(h, router, k, norm)
        assert torch.equal(logits, rlogits)
        assert torch.equal(idx, ridx) and torch.equal(w, rw)
        for a, b in zip(sort, rsort):
            assert torch.equal(a, b)
    oidx, ow = O.route_logits(logits.cpu(), k, norm)
    assert torch.equal(idx.cpu().long(), oidx)
    p = O.plan(oidx, w.cpu(), E)
    counts, offsets, token, wsorted, pos_of = sort
    assert torch.equal(counts.cpu().long(), p.counts) and torch.equal(offsets.cpu().long(), p.offsets)
    assert torch.equal(token.cpu().long(), p.token) and torch.equal(pos_of.cpu().long(), p.pos_of)
    assert torch.equal(wsorted.cpu().view(torch.int16), p.weight.view(torch.int16))


def test_router_route_sort_counters_come_round(K):
    """More launches than the library keeps counters, of two sizes in turn: a launch that finds a
    counter not at zero would sort too early or never."""
    g = torch.Generator().manual_seed(5)
    ext = K.ext()
    cases = []
    for N in (8, 13):
        h = torch.randn(N, 512, generator=g).half().to(DEV)
        router = (torch.randn(64, 512, generator=g) * 512 ** -0.5).half().to(DEV)
        logits = ext.router_logits(h, router)
        idx, w = ext.route(logits, 8, False)
        cases.append((h, router, ext.sort_by_expert(idx, w, 64)))
    results = []
    for i in range(1100):
        h, router, _ = cases[i % 2]
        results.append(ext.router_route_sort(h, router, 8, False)[3:])
    torch.cuda.synchronize()
    for i, got in enumerate(results):
        for a, b in zip(got, cases[i % 2][2]):
            assert torch.equal(a, b), i


def test_captured_router_route_sort_beside_eager_launches(K):
    """A captured launch keeps its counter for every replay, so the library hands captured
    launches counters that no launch outside a capture is ever given: a graph replays on one
    stream while more eager launches than the pool's eager half holds run on another, and every
    replay sorts as the three separate launches do."""
    g = torch.Generator().manual_seed(21)
    ext = K.ext()
    cases = []
    for N in (12, 40):
        h = torch.randn(N, 1024, generator=g).half().to(DEV)
        router = (torch.randn(64, 1024, generator=g) * 1024 ** -0.5).half().to(DEV)
        logits = ext.router_logits(h, router)
        idx, w = ext.route(logits, 8, True)
        cases.append((h, router, [logits, idx, w] + list(ext.sort_by_expert(idx, w, 64))))
    torch.cuda.synchronize()
    side, other = torch.cuda.Stream(), torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        captured = [ext.router_route_sort(cases[0][0], cases[0][1], 8, True) for _ in range(3)]   # three counters
    eager = []
    for rep in range(40):
        with torch.cuda.stream(side):
            graph.replay()
        with torch.cuda.stream(other):
            for _ in range(15):     # 600 in all: the eager half of the pool comes round
                eager.append(ext.router_route_sort(cases[1][0], cases[1][1], 8, True))
        if rep % 8 == 7:
            torch.cuda.synchronize()
            for got in captured:
                for a, b in zip(got, cases[0][2]):
                    assert torch.equal(a, b), rep
    torch.cuda.synchronize()
    for got in captured:
        for a, b in zip(got, cases[0][2]):
            assert torch.equal(a, b)
    for i, got in enumerate(eager):
        for a, b in zip(got, cases[1][2]):
            assert torch.equal(a, b), i


def test_router_route_sort_on_two_streams_at_once(K):
    """Launches on different streams take different counters, so they may run side by side."""
    g = torch.Generator().manual_seed(9)
    ext = K.ext()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    cases = []
    for N in (8, 40):
        h = torch.randn(N, 2048, generator=g).half().to(DEV)
        router = (torch.randn(64, 2048, generator=g) * 2048 ** -0.5).half().to(DEV)
        logits = ext.router_logits(h, router)
        idx, w = ext.route(logits, 8, True)
        cases.append((h, router, [logits, idx, w] + list(ext.sort_by_expert(idx, w, 64))))
    torch.cuda.synchronize()
    results = ([], [])
    for _ in range(60):
        for s in (0, 1):
            with torch.cuda.stream(streams[s]):
                results[s].append(ext.router_route_sort(cases[s][0], cases[s][1], 8, True))
    torch.cuda.synchronize()
    for s in (0, 1):
        for got in results[s]:
            for a, b in zip(got, cases[s][2]):
                assert torch.equal(a, b)


def test_router_route_sort_limits(K):
    h = torch.zeros(4, 256, dtype=torch.float16, device=DEV)
    with pytest.raises(RuntimeError):
        K.ext().router_route_sort(torch.zeros(300, 256, dtype=torch.float16, device=DEV),
                                  torch.zeros(64, 256, dtype=torch.float16, device=DEV), 8, False)   # too many tokens
    with pytest.raises(RuntimeError):
        K.ext().router_route_sort(h, torch.zeros(64, 256, dtype=torch.float16, device=DEV), 9, False)
    with pytest.raises(RuntimeError):
        K.ext().router_route_sort(h, torch.zeros(200, 256, dtype=torch.float16, device=DEV), 8, False)  # too many experts


def test_route_sort_limits(K):
    with pytest.raises(RuntimeError):
        K.ext().route_sort(torch.zeros(300, 64, dtype=torch.float16, device=DEV), 8, False)   # too many tokens
    with pytest.raises(RuntimeError):
        K.ext().route_sort(torch.zeros(4, 64, dtype=torch.float16, device=DEV), 9, False)


@pytest.mark.parametrize("N,E,k,H", [(65, 64, 8, 2048), (1000, 64, 8, 2048), (4096, 64, 8, 2048), (77, 128, 8, 512),
                                     (333, 100, 5, 1024), (16, 8, 2, 512), (1, 64, 8, 512)])
@pytest.mark.parametrize("norm", [False, True])
def test_router_gemm_and_route_in_one_launch(K, N, E, k, H, norm):
    """sy_router_route: logits as the GEMM gives them (to half-precision rounding), and from
    those logits exactly route's ids and weights, which are the oracle's."""
    g = torch.Generator().manual_seed(N + E)
    h = torch.randn(N, H, generator=g).half().to(DEV)
    router = (torch.randn(E, H, generator=g) * H ** -0.5).half().to(DEV)
    idx, w, logits = K.ext().router_route(h, router, k, norm)
    assert torch.allclose(logits.float(), h.float() @ router.float().T, rtol=2 ** -10, atol=1e-3)
    ridx, rw = K.ext().route(logits, k, norm)
    assert torch.equal(idx, ridx) and torch.equal(w, rw)
    oidx, ow = O.route_logits(logits.cpu(), k, norm)
    assert torch.equal(idx.cpu().long(), oidx)
    assert (w.cpu().float() - ow.float()).abs().max().item() < WEIGHT_TOL
    if N >= K.ROUTER_ROUTE_MIN_TOKENS:   # kernels.route takes this launch from there on
        kidx, kw = K.route(h, router, k, norm)
        assert torch.equal(kidx, idx) and torch.equal(kw, w)


def test_router_route_limits(K):
    h = torch.zeros(100, 768, dtype=torch.float16, device=DEV)
    with pytest.raises(RuntimeError):
        K.ext().router_route(h, torch.zeros(64, 768, dtype=torch.float16, device=DEV), 8, False)   # H % 512 != 0
    h = torch.zeros(100, 512, dtype=torch.float16, device=DEV)
    with pytest.raises(RuntimeError):
        K.ext().router_route(h, torch.zeros(200, 512, dtype=torch.float16, device=DEV), 8, False)  # too many experts
    # a layer of that width still runs: the library GEMM makes the logits
    hh, router, gu, dn = (t.to(DEV) for t in cases.layer(100, E=16, k=4, H=768, I=64, seed=1, wstd=0.05))
    out = K.moe_layer(hh, router, gu, dn, 4, False)
    assert out.shape == (100, 768) and torch.isfinite(out.float()).all()


# ------------------------------------------------------------------ the experts of a decode step in one call
@pytest.mark.parametrize("N,E,k,H,I", [(1, 64, 8, 2048, 1024), (8, 64, 8, 2048, 1024), (16, 64, 8, 2048, 1024),
                                       (5, 16, 4, 128, 64), (40, 64, 8, 256, 128), (200, 64, 8, 256, 128),
                                       (3000, 64, 8, 128, 64),         # the sort with a workspace
                                       # router GEMM and route in one launch (H a multiple of 512, above 64 tokens):
                                       (100, 64, 8, 512, 128), (300, 128, 8, 512, 64),
                                       # ... with the router staged through LDS (H >= 1024, E <= 64), one workgroup sorting
                                       (65, 16, 4, 1024, 64), (100, 64, 8, 1024, 64), (250, 60, 8, 1024, 64),
                                       (256, 64, 8, 2048, 64), (511, 64, 4, 1024, 64),
                                       # ... which is also the sort's first pass above 2048 choices
                                       (1100, 64, 8, 512, 64), (2100, 16, 4, 512, 64), (1027, 60, 8, 1024, 64),
                                       # ... with two and four groups of 16 tokens to a piece of the sort
                                       (9000, 64, 8, 512, 64), (33000, 64, 8, 512, 32)])
@pytest.mark.parametrize("tiles", [False, True])
@pytest.mark.parametrize("norm", [False, True])
def test_experts_in_one_call_equal_the_five_calls(K, N, E, k, H, I, tiles, norm):
    """sy_moe_experts enqueues what route_sort, the two projections and combine enqueue: the same
    bits come out, with the weight-stream kernel and with the MFMA tiles; and a layer that
    uses it agrees with the oracle's loop as the layer tests demand."""
    h, router, gu, dn = cases.layer(N, E=E, k=k, H=H, I=I, seed=3, wstd=0.05)
    h, router, gu, dn = (t.to(DEV) for t in (h, router, gu, dn))
    ext = K.ext()
    # the logits the layer itself will route on: the library's own router kernel for tens of tokens
    fused_router = N > K.OWN_ROUTER_MAX_TOKENS and ext.router_route_ok(N, H, E, k)
    if fused_router:
        fidx, fw, logits = ext.router_route(h, router, k, norm)
    else:
        logits = ext.router_logits(h, router) if N <= K.OWN_ROUTER_MAX_TOKENS else F.linear(h, router).contiguous()
    assert torch.allclose(logits.float(), h.float() @ router.float().T, rtol=2 ** -10, atol=1e-4)
    one_launch = N <= K.FUSED_FRONT_MAX_TOKENS
    if one_launch:
        idx, w, counts, offsets, token, wsorted, pos_of = ext.route_sort(logits, k, norm)
    else:
        idx, w = ext.route(logits, k, norm)
        counts, offsets, token, wsorted, pos_of = ext.sort_by_expert(idx, w, E)
    if fused_router:   # the launch that made the logits routed on them as route does
        assert torch.equal(fidx, idx) and torch.equal(fw, w)
    M = N * k
    if tiles:
        act = ext.grouped_gemm(h, token, gu, offsets, None, 0, M, True, None)
        y = ext.grouped_gemm(act, None, dn, offsets, None, 0, M, False, wsorted)
    else:
        act = ext.grouped_gemv(h, token, gu, offsets, M, True, None, N)
        y = ext.grouped_gemv(act, None, dn, offsets, M, False, wsorted, N)
    want = ext.combine(y, pos_of, idx, N)
    got = ext.moe_experts(h, logits, gu, dn, k, norm, mfma_tiles=tiles, one_launch_front=one_launch)
    assert torch.equal(got, want)
    layer = K.moe_layer(h, router, gu, dn, k, norm, mode="gemm" if tiles else "gemv")   # the layer takes this path
    assert torch.equal(layer, want)
    if N <= K.OWN_ROUTER_MAX_TOKENS or fused_router:     # and with the router GEMM inside the same call
        assert torch.equal(ext.moe_experts(h, None, gu, dn, k, norm, mfma_tiles=tiles, one_launch_front=one_launch,
                                           router=router), want)


@pytest.mark.parametrize("N,tiles", [(1, False), (8, False), (40, True), (64, True)])
def test_moe_experts_entry_point_with_a_router_at_decode_sizes(K, N, tiles):
    """The C entry point itself, called as a foreign binding would (one call, the router given):
    up to 64 tokens it runs the one-launch front, which the Python binding enqueues separately."""
    E, k, H, I = 64, 8, 512, 128
    h, router, gu, dn = (t.to(DEV) for t in cases.layer(N, E=E, k=k, H=H, I=I, seed=4, wstd=0.05))
    ext = K.ext()
    want = K.moe_layer(h, router, gu, dn, k, True, mode="gemm" if tiles else "gemv")
    M = N * k
    i32 = dict(dtype=torch.int32, device=DEV)
    f16 = dict(dtype=torch.float16, device=DEV)
    logits, idx, w = torch.empty(N, E, **f16), torch.empty(N, k, **i32), torch.empty(N, k, **f16)
    counts, offsets = torch.empty(E, **i32), torch.empty(E + 1, **i32)
    token, wsorted, pos_of = torch.empty(M, **i32), torch.empty(M, **f16), torch.empty(M, **i32)
    act, y, out = torch.empty(M, I, **f16), torch.empty(M, H, **f16), torch.empty(N, H, **f16)
    rc = ext.lib.sy_moe_experts(h.data_ptr(), router.data_ptr(), logits.data_ptr(), N, E, k, 1, gu.data_ptr(), dn.data_ptr(),
                                H, I, int(tiles), 0, idx.data_ptr(), w.data_ptr(), counts.data_ptr(), offsets.data_ptr(),
                                token.data_ptr(), wsorted.data_ptr(), pos_of.data_ptr(), act.data_ptr(), y.data_ptr(),
                                out.data_ptr(), None, 0, torch.cuda.current_stream().cuda_stream)
    assert rc == 0, ext.lib.sy_last_error()
    assert torch.equal(out, want)
    assert torch.equal(logits, ext.router_logits(h, router))
    ridx, rw = ext.route(logits, k, True)
    assert torch.equal(idx, ridx) and torch.equal(w, rw)
    for a, b in zip((counts, offsets, token, wsorted, pos_of), ext.sort_by_expert(ridx, rw, E)):
        assert torch.equal(a, b)


@pytest.mark.parametrize("N,E,k,H,I", [(1, 64, 8, 2048, 1024), (8, 64, 8, 2048, 1024), (5, 16, 4, 128, 64), (3, 128, 8, 520, 72),
                                       (64, 64, 1, 256, 128), (7, 60, 3, 1024, 256),
                                       (9, 64, 8, 512, 128), (300, 64, 8, 256, 128)])   # these two sort in a launch of their own
@pytest.mark.parametrize("tiles", [False, True])
def test_experts_from_the_routing_in_one_call(K, N, E, k, H, I, tiles):
    """sy_experts_routed is experts() of the reference in one call. Up to 64 choices on the
    weight-stream kernels the gate/up launch sorts for itself: the sort's five results and
    `out` are bit for bit those of sort_by_expert, the two projections and combine."""
    if tiles and (H % 32 or I % 32):
        pytest.skip("the MFMA tiles need K % 32 == 0, as the reference's do")
    h, router, gu, dn = (t.to(DEV) for t in cases.layer(N, E=E, k=k, H=H, I=I, seed=6, wstd=0.05))
    ext = K.ext()
    idx, w = ext.route(F.linear(h, router).contiguous(), k, True)
    want_sort = ext.sort_by_expert(idx, w, E)
    counts, offsets, token, wsorted, pos_of = want_sort
    want = ext.combine(K.ffn(h, token, offsets, counts, wsorted, gu, dn, N * k, "gemm" if tiles else "gemv"), pos_of, idx, N)
    assert torch.equal(K.experts(h, idx, w, gu, dn, "gemm" if tiles else "gemv"), want)   # experts() takes the one call
    M = N * k
    i32 = dict(dtype=torch.int32, device=DEV)
    f16 = dict(dtype=torch.float16, device=DEV)
    counts, offsets = torch.empty(E, **i32), torch.empty(E + 1, **i32)
    token, wsorted, pos_of = torch.empty(M, **i32), torch.empty(M, **f16), torch.empty(M, **i32)
    act, y, out = torch.empty(M, I, **f16), torch.empty(M, H, **f16), torch.empty(N, H, **f16)
    need = ext.lib.sy_sort_workspace_bytes(N, k, E)
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=DEV)
    for _ in range(2):
        rc = ext.lib.sy_experts_routed(h.data_ptr(), N, E, k, gu.data_ptr(), dn.data_ptr(), H, I, int(tiles), idx.data_ptr(),
                                       w.data_ptr(), counts.data_ptr(), offsets.data_ptr(), token.data_ptr(),
                                       wsorted.data_ptr(), pos_of.data_ptr(), act.data_ptr(), y.data_ptr(), out.data_ptr(),
                                       ws.data_ptr(), need, torch.cuda.current_stream().cuda_stream)
        assert rc == 0, ext.lib.sy_last_error()
        assert torch.equal(out, want)
        for a, b in zip((counts, offsets, token, wsorted, pos_of), want_sort):
            assert torch.equal(a, b)


@pytest.mark.parametrize("N,E,k,H,I,routing", [(2, 64, 8, 2048, 1024, "routed"), (3, 64, 8, 2048, 1024, "routed"),
                                               (4, 64, 8, 2048, 1024, "routed"), (4, 16, 4, 256, 512, "routed"),
                                               (3, 128, 8, 512, 1024, "routed"), (4, 8, 8, 1024, 512, "routed"),
                                               (4, 64, 8, 2048, 1024, "one expert"), (4, 16, 8, 256, 512, "two experts"),
                                               (1, 4, 4, 8, 512, "routed")])
def test_down_projection_and_combine_in_one_launch(K, N, E, k, H, I, routing):
    """Up to 4 tokens (32 sorted rows) on the weight-stream kernels sy_experts_routed ends in one
    launch that projects down and adds each token's rows up: `out` has the bits of the down
    projection without scales followed by the combine that applies the router weights, and of
    the plain separate calls. With ids that repeat inside a token (experts() takes any idx) an
    expert has up to 32 rows."""
    h, router, gu, dn = (t.to(DEV) for t in cases.layer(N, E=E, k=k, H=H, I=I, seed=12, wstd=0.05))
    ext = K.ext()
    assert ext.lib.sy_version() >= 200
    idx, w = ext.route(F.linear(h, router).contiguous(), k, True)
    if routing == "one expert":
        idx = torch.full_like(idx, 5)
    elif routing == "two experts":
        idx = (torch.arange(N * k, device=DEV, dtype=torch.int32).reshape(N, k) % 2) * 9 + 3
    counts, offsets, token, wsorted, pos_of = ext.sort_by_expert(idx, w, E)
    M = N * k
    act = ext.grouped_gemv(h, token, gu, offsets, M, True, None, M)
    want = ext.combine(ext.grouped_gemv(act, None, dn, offsets, M, False, wsorted, M), pos_of, idx, N)
    for _ in range(2):
        assert torch.equal(ext.experts_routed(h, idx, w, gu, dn, mfma_tiles=False), want)
    oracle = O.experts_loop(h.cpu().float(), idx.cpu().long(), w.cpu().float(), gu.cpu().float(), dn.cpu().float())
    assert (want.cpu().float() - oracle).abs().max().item() <= 2e-2


@pytest.mark.parametrize("N,E,k,H", [(1, 64, 8, 2048), (8, 64, 8, 2048), (64, 64, 8, 2048), (5, 100, 5, 520), (64, 128, 8, 8192)])
def test_router_route_at_decode_sizes(K, N, E, k, H):
    """Up to 64 tokens sy_router_route is a workgroup per token: the logits of router_logits and
    the ids and weights of route on them, bit for bit."""
    g = torch.Generator().manual_seed(N + E)
    h = torch.randn(N, H, generator=g).half().to(DEV)
    router = (torch.randn(E, H, generator=g) * H ** -0.5).half().to(DEV)
    ext = K.ext()
    idx, w, logits = ext.router_route(h, router, k, True)
    assert torch.equal(logits, ext.router_logits(h, router))
    ridx, rw = ext.route(logits, k, True)
    assert torch.equal(idx, ridx) and torch.equal(w, rw)


def test_moe_experts_entry_point_with_a_width_the_mfma_front_does_not_take(K):
    """A foreign binding that gives the router for 100 tokens of width 768 (not a multiple of
    512): the call makes the logits with the row kernel and routes and sorts in launches of
    their own, with the results of the separate entry points."""
    N, E, k, H, I = 100, 16, 4, 768, 64
    h, router, gu, dn = (t.to(DEV) for t in cases.layer(N, E=E, k=k, H=H, I=I, seed=6, wstd=0.05))
    ext = K.ext()
    assert not ext.router_route_ok(N, H, E, k)
    M = N * k
    i32 = dict(dtype=torch.int32, device=DEV)
    f16 = dict(dtype=torch.float16, device=DEV)
    logits, idx, w = torch.empty(N, E, **f16), torch.empty(N, k, **i32), torch.empty(N, k, **f16)
    counts, offsets = torch.empty(E, **i32), torch.empty(E + 1, **i32)
    token, wsorted, pos_of = torch.empty(M, **i32), torch.empty(M, **f16), torch.empty(M, **i32)
    act, y, out = torch.empty(M, I, **f16), torch.empty(M, H, **f16), torch.empty(N, H, **f16)
    need = ext.lib.sy_sort_workspace_bytes(N, k, E)
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=DEV)
    for tiles in (0, 1):
        rc = ext.lib.sy_moe_experts(h.data_ptr(), router.data_ptr(), logits.data_ptr(), N, E, k, 0, gu.data_ptr(),
                                    dn.data_ptr(), H, I, tiles, 0, idx.data_ptr(), w.data_ptr(), counts.data_ptr(),
                                    offsets.data_ptr(), token.data_ptr(), wsorted.data_ptr(), pos_of.data_ptr(),
                                    act.data_ptr(), y.data_ptr(), out.data_ptr(), ws.data_ptr(), need,
                                    torch.cuda.current_stream().cuda_stream)
        assert rc == 0, ext.lib.sy_last_error()
        assert torch.equal(logits, ext.router_logits(h, router))
        ridx, rw = ext.route(logits, k, False)
        assert torch.equal(idx, ridx) and torch.equal(w, rw)
        oidx, _ = O.route_logits(logits.cpu(), k, False)
        assert torch.equal(idx.cpu().long(), oidx)
        assert torch.equal(out, K.experts(h, ridx, rw, gu, dn, "gemm" if tiles else "gemv"))


@pytest.mark.parametrize("path", ["layer", "experts"])
def test_a_captured_layer_keeps_its_scratch_while_other_shapes_come_and_go(K, path):
    """The binding keeps the intermediate results of small calls per (shape, stream) and drops the
    least recently used of them. A HIP graph captured through the call has the allocation's
    address in its kernel arguments, so that allocation must outlive any number of other shapes:
    capture a layer of 8 tokens, run more other shapes than the binding keeps, replay. Both
    bindings that keep scratch: moe_layer (one call of the library, the router given) and
    moe_experts (the logits given)."""
    E, k, H, I = 64, 8, 512, 128
    _, router, gu, dn = (t.to(DEV) for t in cases.layer(1, E=E, k=k, H=H, I=I, seed=8, wstd=0.05))
    ext = K.ext()
    if path == "layer":
        call = lambda x: K.moe_layer(x, router, gu, dn, k, False)
        pinned, kept_lru = (lambda: len(ext._scratch_pinned)), (lambda: len(ext._scratch))
    else:
        call = lambda x: ext.moe_experts(x, F.linear(x, router).contiguous(), gu, dn, k, False, one_launch_front=True)
        pinned, kept_lru = (lambda: len(ext._captured)), (lambda: len(ext._plans))
    h = hidden(8, H)
    want = call(h).clone()
    static_h = h.clone()
    torch.cuda.synchronize()
    before = pinned()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = call(static_h)
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(captured, want)
    kept = pinned()
    assert kept >= max(before, 1)
    others = []
    for n in range(9, 9 + ext.PLANS_MAX + 4):     # more shapes than the binding keeps
        others.append(call(hidden(n, H)))
    big = [torch.empty(32 << 20, dtype=torch.uint8, device=DEV).fill_(0xff) for _ in range(8)]   # reuse freed memory, if any
    torch.cuda.synchronize()
    assert kept_lru() <= ext.PLANS_MAX and pinned() == kept
    for seed in (1, 2):
        static_h.copy_(hidden(8, H, seed=seed))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(captured, call(static_h))
    del big, others


def test_the_layer_in_one_call_equals_the_separate_calls(K):
    """sy_moe_layer (one description of the layer, one scratch buffer) against route, sort, the
    two projections and combine called one by one, at a decode size, at a size of the MFMA
    tiles and at a width the MFMA front does not take; and the raw entry point refuses a
    scratch buffer that is too small."""
    ext = K.ext()
    for N, E, k, H, I, mode in ((8, 64, 8, 512, 128, "gemv"), (3, 16, 4, 128, 64, "gemv"), (40, 64, 8, 512, 128, "gemm"),
                                (300, 64, 8, 512, 64, "gemm"), (100, 16, 4, 768, 64, "gemm")):
        h, router, gu, dn = (t.to(DEV) for t in cases.layer(N, E=E, k=k, H=H, I=I, seed=11, wstd=0.05))
        got = ext.moe_layer(h, router, gu, dn, k, True, mode != "gemv")
        if N <= K.OWN_ROUTER_MAX_TOKENS or not ext.router_route_ok(N, H, E, k):
            logits = ext.router_logits(h, router)
        else:
            _, _, logits = ext.router_route(h, router, k, True)
        idx, w = ext.route(logits, k, True)
        assert torch.equal(got, K.experts(h, idx, w, gu, dn, mode)), (N, E, H, mode)
        oidx, _ = O.route_logits(logits.cpu(), k, True)
        assert torch.equal(idx.cpu().long(), oidx)
    from switchyard_amd._abi import SyMoeLayer
    need = ext.lib.sy_moe_layer_scratch_bytes(N, E, k, H, I)
    small = torch.empty(need - 256, dtype=torch.uint8, device=DEV)
    out = torch.empty_like(h)
    desc = SyMoeLayer(N, E, k, 1, H, I, 1, 0, router.data_ptr(), gu.data_ptr(), dn.data_ptr(), small.data_ptr(), small.numel())
    assert ext.lib.sy_moe_layer(desc, h.data_ptr(), out.data_ptr(), torch.cuda.current_stream().cuda_stream) == 1
    assert b"scratch" in ext.lib.sy_last_error()

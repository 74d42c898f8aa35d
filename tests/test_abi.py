"""The C-ABI library loads without a GPU, exports every symbol the header declares, and
rejects out-of-range arguments before touching the device. No compute is launched here."""

import ctypes
import os
import re

import pytest

from switchyard_amd import _abi, kernels

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "switchyard_moe.h")
DECODE_HEADER = os.path.join(ROOT, "include", "switchyard_decode.h")


@pytest.fixture(scope="module")
def lib():
    return _abi.load_library()


def declared_symbols(header=None):
    text = open(header).read() if header else open(HEADER).read() + open(DECODE_HEADER).read()
    return re.findall(r"^SY_API\s+[\w\s\*]+?\b(sy_\w+)\(", text, flags=re.M)


def test_header_declares_the_expected_entry_points():
    assert sorted(declared_symbols(DECODE_HEADER)) == ["sy_add_rmsnorm", "sy_add_rmsnorm_logits", "sy_add_rmsnorm_route_sort",
                                                           "sy_combine_add_rmsnorm",
                                                       "sy_decode_attention", "sy_decode_attention_qkv", "sy_embed_rmsnorm",
                                                       "sy_greedy_advance", "sy_qk_norm_rope_cache", "sy_router_logits",
                                                           "sy_router_route_sort"]
    assert sorted(os.listdir(os.path.join(ROOT, "include"))) == ["switchyard_decode.h", "switchyard_moe.h"]
    assert sorted(declared_symbols(HEADER)) == sorted(["sy_version", "sy_last_error", "sy_route", "sy_sort_workspace_bytes",
                                                  "sy_sort_by_expert", "sy_sort_by_expert_static", "sy_route_sort", "sy_router_route", "sy_experts_sorted", "sy_experts_routed",
                                                  "sy_grouped_gemv", "sy_grouped_gemv_sorting", "sy_grouped_gemm",
                                                  "sy_combine", "sy_moe_experts", "sy_moe_layer", "sy_moe_layer_scratch_bytes"])


def test_library_exports_every_declared_symbol(lib):
    raw = ctypes.CDLL(_abi.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(raw, name), name
        assert name in _abi.SIGNATURES, f"{name} has no ctypes signature"
    assert lib.sy_version() >= 100


def test_each_header_citation_names_a_reference_location():
    text = open(HEADER).read()
    for name in ("sy_route", "sy_sort_by_expert", "sy_route_sort", "sy_grouped_gemv", "sy_grouped_gemv_sorting", "sy_grouped_gemm",
                 "sy_combine",
                 "sy_moe_experts", "sy_moe_layer"):
        comment = text[:text.index(f"SY_API int {name}(")].rsplit("/*", 1)[1]
        assert re.search(r"(moe_kernels\.cu|kernels\.py):\d+", comment), name
    # the entry point that allocates nothing replaces no reference interface and says so
    comment = text[:text.index("SY_API int sy_sort_by_expert_static(")].rsplit("/*", 1)[1]
    assert "no counterpart in the reference" in comment and "cannot allocate" in comment
    assert not re.search(r"(moe_kernels\.cu|kernels\.py):\d+", comment)


def test_each_decode_citation_names_a_reference_location():
    text = open(DECODE_HEADER).read()
    for name in declared_symbols(DECODE_HEADER):
        comment = text[:text.index(f"SY_API int {name}(")].rsplit("/*", 1)[1]
        assert re.search(r"(model|kernels)\.py:\d+", comment), name


def test_decode_argument_errors_and_empty_batches(lib):
    assert lib.sy_add_rmsnorm(None, None, None, 1e-5, 4, 2052, None, None, None) == 1
    assert b"multiple of 8" in lib.sy_last_error()
    assert lib.sy_add_rmsnorm(None, None, None, 1e-5, 4, 16384, None, None, None) == 1
    assert lib.sy_add_rmsnorm(None, None, None, 1e-5, 0, 2048, None, None, None) == 0
    assert lib.sy_embed_rmsnorm(None, None, 0, None, 1e-5, 4, 2048, None, None, None) == 1
    assert lib.sy_embed_rmsnorm(None, None, 100, None, 1e-5, 0, 2048, None, None, None) == 0
    assert lib.sy_greedy_advance(None, 4, 0, None, None, 8, None, None, None, None) == 1
    assert lib.sy_greedy_advance(None, 0, 1000, None, None, 8, None, None, None, None) == 0
    assert lib.sy_greedy_advance(None, 4, 1000, None, None, 8, None, None, None, None) == 1   # null pointers
    assert lib.sy_add_rmsnorm_logits(None, None, None, 1e-5, None, 2000, 4, 2048, None, None, None, None) == 1
    assert lib.sy_add_rmsnorm_logits(None, None, None, 1e-5, None, 64, 0, 2048, None, None, None, None) == 0
    assert lib.sy_combine_add_rmsnorm(None, None, None, None, 65, None, None, 1e-5, 4, 2048, None, None, None) == 1
    assert lib.sy_combine_add_rmsnorm(None, None, None, None, 8, None, None, 1e-5, 4, 2044, None, None, None) == 1
    assert lib.sy_combine_add_rmsnorm(None, None, None, None, 8, None, None, 1e-5, 0, 2048, None, None, None) == 0
    nine = (None,) * 9
    assert lib.sy_router_route_sort(None, None, 0, 2048, 64, 8, 0, *nine) == 0
    assert lib.sy_router_route_sort(None, None, 4, 2044, 64, 8, 0, *nine) == 1
    assert lib.sy_router_route_sort(None, None, 4, 2048, 64, 8, 0, *nine) == 1          # null pointers
    assert lib.sy_add_rmsnorm_route_sort(None, None, None, 1e-5, None, 64, 0, 2048, 8, 0, *nine, None, None) == 0
    assert lib.sy_add_rmsnorm_route_sort(None, None, None, 1e-5, None, 64, 4, 2048, 8, 0, *nine, None, None) == 1
    assert lib.sy_qk_norm_rope_cache(None, None, None, 1e-5, 0.0, None, None, 64, None, None, 2, 1, 16, 5, 128, 64, None,
                                     None, None, None) == 1
    assert lib.sy_qk_norm_rope_cache(None, None, None, 1e-5, 0.0, None, None, 64, None, None, 2, 1, 16, 16, 72, 64, None,
                                     None, None, None) == 1
    assert lib.sy_qk_norm_rope_cache(None, None, None, 1e-5, 0.0, None, None, 64, None, None, 2, 0, 16, 16, 128, 64, None,
                                     None, None, None) == 1
    assert lib.sy_qk_norm_rope_cache(None, None, None, 1e-5, 0.0, None, None, 64, None, None, 0, 1, 16, 16, 128, 64, None,
                                     None, None, None) == 0
    assert lib.sy_decode_attention(None, None, None, None, None, 2, 16, 16, 96, 64, None, None) == 1
    assert b"64 or 128" in lib.sy_last_error()
    assert lib.sy_decode_attention(None, None, None, None, None, 2, 16, 3, 128, 64, None, None) == 1
    assert lib.sy_decode_attention(None, None, None, None, None, 0, 16, 16, 128, 64, None, None) == 0
    assert lib.sy_decode_attention(None, None, None, None, None, 2, 16, 16, 128, 64, None, None) == 1  # null pointers


def test_argument_errors_are_reported_without_a_device(lib):
    assert lib.sy_route(None, 0, 5, 200, 8, 0, None, None, None) == 1
    assert b"128 experts" in lib.sy_last_error()
    assert lib.sy_route(None, 0, 5, 64, 9, 0, None, None, None) == 1
    assert lib.sy_route(None, 7, 5, 64, 8, 0, None, None, None) == 1
    assert lib.sy_grouped_gemm(None, None, None, None, 64, 5, 1024, 2040, 1, None, None, None) == 1
    assert b"multiple of 32" in lib.sy_last_error()
    assert lib.sy_grouped_gemv(None, None, None, None, 64, 5, 0, 1024, 2044, 1, None, None, None) == 1
    assert lib.sy_combine(None, None, None, 4, 8, 2044, None, None) == 1
    assert lib.sy_combine(None, None, None, 4, 65, 2048, None, None) == 1
    assert lib.sy_sort_by_expert(None, None, 3, 4, 8, 64, None, None, None, None, None, None, 0, None) == 1
    assert lib.sy_sort_by_expert(None, None, 2, 4, 8, 513, None, None, None, None, None, None, 0, None) == 1
    # the static array holds 1 MiB of histograms: 160 000 choices over 512 experts need more
    assert lib.sy_sort_workspace_bytes(20000, 8, 512) > (1 << 20)
    assert lib.sy_sort_by_expert_static(None, None, 2, 20000, 8, 512, None, None, None, None, None, None) == 1
    assert b"static" in lib.sy_last_error()
    assert lib.sy_sort_by_expert_static(None, None, 3, 4, 8, 64, None, None, None, None, None, None) == 1


def test_empty_inputs_are_no_ops(lib):
    assert lib.sy_route(None, 0, 0, 64, 8, 0, None, None, None) == 0
    assert lib.sy_grouped_gemv(None, None, None, None, 64, 0, 0, 1024, 2048, 1, None, None, None) == 0
    assert lib.sy_grouped_gemm(None, None, None, None, 64, 0, 1024, 2048, 1, None, None, None) == 0
    assert lib.sy_combine(None, None, None, 0, 8, 2048, None, None) == 0


def test_sort_workspace_grows_with_the_number_of_choices(lib):
    assert lib.sy_sort_workspace_bytes(8, 8, 64) == 0
    big = lib.sy_sort_workspace_bytes(4096, 8, 64)
    assert big > 0 and lib.sy_sort_workspace_bytes(32768, 8, 64) > big


def test_pick_and_tile_offsets_host_logic():
    import torch

    assert kernels.pick(1) == "gemv" and kernels.pick(kernels.GEMV_MAX_ROWS) == "gemv"
    assert kernels.pick(kernels.GEMV_MAX_ROWS + 1) == "gemm" and kernels.pick(10 ** 6) == "gemm"
    assert kernels._auto(8, 64, 64) == "gemv" and kernels._auto(4096, 32768, 64) == "gemm"
    counts = torch.tensor([0, 1, 64, 65, 128, 0, 200])
    assert kernels.tile_offsets(counts).tolist() == [0, 0, 1, 2, 4, 6, 6, 10]


def test_host_wrappers_refuse_cpu_tensors():
    import torch

    with pytest.raises(RuntimeError, match="contiguous GPU tensor"):
        kernels.ext().route(torch.zeros(4, 64, dtype=torch.float16), 8, False)
    with pytest.raises(ValueError, match="unknown mode"):
        kernels.ffn(torch.zeros(1, 8), None, None, None, None, None, torch.zeros(1, 8, 8), 1, "nope")


def test_bench_refuses_more_than_one_gpu_and_needs_a_gpu():
    """The benchmark is a one-GPU measurement: --gpus 2 ends with a message, before any device
    is touched; without a GPU the default run says so instead of falling back to the CPU."""
    import subprocess
    import sys

    bench = os.path.join(ROOT, "bench.py")
    two = subprocess.run([sys.executable, bench, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert two.returncode != 0 and "one GPU" in two.stderr
    import torch

    if not torch.cuda.is_available():
        one = subprocess.run([sys.executable, bench], capture_output=True, text=True, timeout=120)
        assert one.returncode != 0 and "no GPU" in one.stderr


def test_the_reference_module_path_serves_the_same_names_and_signatures():
    """`from switchyard import kernels` is the reference's import (switchyard/kernels.py:12-93);
    the parameters and defaults below are the reference's, and `ext()` offers the five methods of
    its native module that the one-GPU path uses (moe_kernels.cu:491-495) with their arguments
    (:73, :142, :264-266, :385-386, :435)."""
    import inspect

    from switchyard import kernels as drop_in

    assert drop_in.moe_layer is kernels.moe_layer and drop_in.ext is kernels.ext
    want = {
        "ext": [],
        "tile_offsets": ["counts", ("block", 64)],
        "route": ["h", "router", "top_k", "norm_topk_prob"],
        "pick": ["max_rows"],
        "ffn": ["x", "a_rows", "offsets", "counts", "wsorted", "gate_up", "down", "rows", "mode", ("host_counts", None)],
        "experts": ["h", "idx", "w", "gate_up", "down", ("mode", "auto")],
        "moe_layer": ["h", "router", "gate_up", "down", "top_k", "norm_topk_prob", ("mode", "auto")],
    }
    for name, params in want.items():
        sig = inspect.signature(getattr(drop_in, name))
        got = [(p.name, p.default) if p.default is not inspect.Parameter.empty else p.name for p in sig.parameters.values()]
        assert got == params, name
    assert isinstance(drop_in.GEMV_MAX_ROWS, int) and isinstance(drop_in.GEMM_MAX_ROWS, int)
    assert sorted(drop_in.__all__) == sorted(list(want) + ["GEMV_MAX_ROWS", "GEMM_MAX_ROWS"])
    native = {
        "route": ["logits", "k", "norm"],
        "sort_by_expert": ["idx", "w", "E"],
        "grouped_gemm": ["A", "a_rows", "B", "offsets", "tile_offsets", "total_tiles", "rows", "swiglu", "scale"],
        "grouped_gemv": ["A", "a_rows", "B", "offsets", "rows", "swiglu", "scale"],
        "combine": ["y", "pos_of", "idx", "n_tokens"],
    }
    for name, params in native.items():
        sig = inspect.signature(getattr(_abi.Ext, name))
        required = [p.name for p in sig.parameters.values() if p.name != "self" and p.default is inspect.Parameter.empty]
        assert required == params, name

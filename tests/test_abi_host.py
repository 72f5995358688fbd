"""Host-only checks of the drop-in boundary: both libraries load, export every
symbol include/*.h declares, and turn invalid arguments into status 1 plus the
reference's message without touching a GPU (validation precedes any runtime
call, as in the reference: kernels/attention/mla/sm89.cu:20-24,514)."""

import ctypes
import re
from pathlib import Path

import pytest

from dscuda_amd.harness.common import F, I, P, ROOT, bind, checked, library, library_path


def _declared_symbols(header):
    text = (ROOT / "include" / header).read_text()
    block = text[text.index('extern "C" {'):]
    return sorted(set(re.findall(r"\b(dscuda_\w+)\s*\(", block)))


def test_libraries_exist_under_build():
    # file names are part of the contract (benchmarks/common.py:19-20)
    assert library_path("mla").name == "libdscuda_mla_bench.so"
    assert library_path("flash_attention").name == "libdscuda_flash_attention_bench.so"
    assert library_path("mla").exists() and library_path("flash_attention").exists()


@pytest.mark.parametrize("name,header", [("mla", "mla.h"), ("flash_attention", "flash_attention.h")])
def test_every_declared_symbol_is_exported(name, header):
    lib = library(name)
    symbols = _declared_symbols(header)
    assert symbols, header
    for symbol in symbols:
        assert getattr(lib, symbol) is not None, symbol
    if name == "mla":
        assert {"dscuda_mla_forward", "dscuda_mla_backward", "dscuda_mla_decode", "dscuda_mla_workspace_elements",
                "dscuda_mla_last_error", "dscuda_mla_prefill_forward", "dscuda_mla_prefill_backward",
                "dscuda_mla_prefill_backward_workspace_elements"} <= set(symbols)
    else:
        assert {"dscuda_flash_forward", "dscuda_flash_last_error"} <= set(symbols)


def test_workspace_elements_match_the_reference_formula():
    lib = library("mla")
    size = bind(lib, "dscuda_mla_workspace_elements", [I] * 4, ctypes.c_size_t)
    assert size(2, 3, 8, 512) == 2 * 3 * 8 * 514          # kernels/attention/mla/sm89.cu:539-541
    assert size(64, 128, 8, 512) == 64 * 128 * 8 * 514
    assert size(4096, 128, 64, 512) == 4096 * 128 * 64 * 514  # needs size_t
    prefill = bind(lib, "dscuda_mla_prefill_backward_workspace_elements", [I] * 5, ctypes.c_size_t)
    # per (batch, head): 128 floats of row statistics per 64-query tile, plus one 16 KB bf16 dS
    # block (4096 floats) per (128-key block, 64-query tile) pair on or below the diagonal
    assert prefill(1, 4096, 128, 192, 128) == 128 * (64 * 128 + (32 * 64 - 32 * 31) * 4096)
    assert prefill(2, 65, 3, 192, 128) == 2 * 3 * (2 * 128 + 2 * 4096)   # ragged: 1 key block, 2 query tiles
    assert prefill(0, 65, 3, 192, 128) == 0


def test_size_queries_need_no_device():
    """Every size query is arithmetic on its integer arguments (benchmarks/bindings/mla_bridge.cu:53-56 is): on a host
    without a GPU it returns, in a process of its own so that an exception let through the C boundary shows up as a
    failed status here instead of ending the test run."""
    import subprocess
    import sys
    script = """
import ctypes, sys
from dscuda_amd.harness.common import I, bind, library
mla, flash = library("mla"), library("flash_attention")
size_t = ctypes.c_size_t
plan = bind(mla, "dscuda_mla_decode_plan_elements", [I] * 4, size_t)
assert plan(2, 3, 8, 512) == 5 + 2 + 1 + 1024, plan(2, 3, 8, 512)        # header, prefix, one entry per range
assert plan(64, 128, 8, 512) == 5 + 64 + 1 + 1024
assert plan(3500, 128, 8, 512) == 5 + 3500 + 1 + 3500                    # one workgroup per sequence at most
assert plan(2, 3, 8, 256) == 0 and plan(0, 3, 8, 512) == 0 and plan(2, 3, 0, 512) == 0
assert bind(mla, "dscuda_mla_workspace_elements", [I] * 4, size_t)(2, 3, 8, 512) == 2 * 3 * 8 * 514
prefill = bind(mla, "dscuda_mla_prefill_backward_workspace_elements", [I] * 5, size_t)
assert prefill(2, 65, 3, 192, 128) == 2 * 3 * (2 * 128 + 2 * 4096) and prefill(1, -4, 3, 192, 128) == 0
backward = bind(flash, "dscuda_flash_backward_workspace_elements", [I] * 5, size_t)
assert backward(1, 128, 4, 2, 64) > 0
assert backward(1, 128, 4, 3, 64) == 0 and backward(1, 128, 4, 0, 64) == 0 and backward(1, 128, 4, 2, 96) == 0
limit = bind(mla, "dscuda_mla_prefill_backward_set_workspace_limit", [size_t], None)
limit(3 * 16384)                                                        # room for three dS blocks: one pair at a time
assert prefill(2, 65, 3, 192, 128) == 2 * 3 * 2 * 128 + 2 * 4096
limit(0)
assert prefill(2, 65, 3, 192, 128) == 2 * 3 * (2 * 128 + 2 * 4096)
bind(mla, "dscuda_mla_backward_set_key_interval_tiles", [I], None)(7)
bind(flash, "dscuda_flash_backward_set_workspace_limit", [size_t], None)(0)
print("size queries ok")
"""
    result = subprocess.run([sys.executable, "-c", script], cwd=ROOT, capture_output=True, text=True, timeout=120)
    assert result.returncode == 0 and "size queries ok" in result.stdout, result.stdout + result.stderr


def _status_and_message(lib, prefix, status):
    with pytest.raises(RuntimeError) as info:
        checked(lib, prefix, status)
    return str(info.value)


def test_mla_shape_errors_round_trip_without_a_gpu():
    lib = library("mla")
    forward = bind(lib, "dscuda_mla_forward", [P] * 6 + [I] * 5 + [F, P])
    backward = bind(lib, "dscuda_mla_backward", [P] * 11 + [I] * 5 + [F, P])
    decode = bind(lib, "dscuda_mla_decode", [P] * 7 + [I] * 7 + [F, P])
    null = [None]
    assert _status_and_message(lib, "mla", forward(*null * 6, 1, 8, 2, 256, 64, 1.0, None)) == \
        "MLA requires C=512 and RoPE=64"
    assert _status_and_message(lib, "mla", backward(*null * 11, 1, 8, 2, 512, 32, 1.0, None)) == \
        "MLA requires C=512 and RoPE=64"
    assert _status_and_message(lib, "mla", decode(*null * 7, 1, 8, 128, 64, 64, 4, 8, 1.0, None)) == \
        "MLA requires C=512 and RoPE=64"
    assert "positive" in _status_and_message(lib, "mla", forward(*null * 6, 0, 8, 2, 512, 64, 1.0, None))
    assert "positive" in _status_and_message(lib, "mla", decode(*null * 7, 1, 8, 512, 64, 64, 4, 0, 1.0, None))
    # the backward keeps intermediate values in its query-gradient outputs: 16-byte alignment is checked first
    misaligned = [0x1008, 0x2000] + [0x3000] * 9
    assert "aligned to 16 bytes" in _status_and_message(lib, "mla", backward(*misaligned, 1, 8, 2, 512, 64, 1.0, None))
    prefill = bind(lib, "dscuda_mla_prefill_forward", [P] * 5 + [I] * 5 + [F, P])
    assert "(d_qk,d_v)" in _status_and_message(lib, "mla", prefill(*null * 5, 1, 8, 2, 96, 96, 1.0, None))
    prefill_backward = bind(lib, "dscuda_mla_prefill_backward", [P] * 10 + [I] * 5 + [F, P])
    assert "workspace" in _status_and_message(
        lib, "mla", prefill_backward(*null * 10, 1, 8, 2, 192, 128, 1.0, None))


def test_flash_errors_round_trip_without_a_gpu():
    lib = library("flash_attention")
    forward = bind(lib, "dscuda_flash_forward", [P] * 5 + [I] * 5 + [F, P])
    null = [None]
    # messages of kernels/attention/flash_attention/sm89_forward.cu:226-232 (head-size rule widened to 64 | 128)
    assert _status_and_message(lib, "flash", forward(*null * 5, 1, 64, 2, 2, 96, 1.0, None)) == \
        "flash attention requires head_size = 64 or 128"
    assert _status_and_message(lib, "flash", forward(*null * 5, 1, 65, 2, 2, 128, 1.0, None)) == \
        "flash attention requires T to be a positive multiple of 64"
    assert _status_and_message(lib, "flash", forward(*null * 5, 1, 0, 2, 2, 128, 1.0, None)) == \
        "flash attention requires T to be a positive multiple of 64"
    assert _status_and_message(lib, "flash", forward(*null * 5, 1, 64, 3, 2, 128, 1.0, None)) == \
        "flash attention requires query_heads to be divisible by key_value_heads"


def test_last_error_is_per_thread_and_sticky():
    import threading
    lib = library("mla")
    forward = bind(lib, "dscuda_mla_forward", [P] * 6 + [I] * 5 + [F, P])
    last = bind(lib, "dscuda_mla_last_error", [], ctypes.c_char_p)
    assert forward(*[None] * 6, 1, 8, 2, 100, 64, 1.0, None) == 1
    first = last().decode()
    seen = {}

    def other():
        seen["before"] = last().decode()   # a fresh thread has no error yet

    thread = threading.Thread(target=other)
    thread.start()
    thread.join()
    assert first == "MLA requires C=512 and RoPE=64" and seen["before"] == ""
    assert last().decode() == first        # still there until the next error on this thread


def test_ops_refuse_cpu_tensors():
    import torch
    from dscuda_amd.harness import ops
    q = torch.zeros(1, 64, 2, 128, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="no CPU path"):
        ops.flash_forward(q, q, q, 1.0)

"""Every C-ABI entry point against the committed golden fixtures."""

import pytest
import torch

from dscuda_amd.harness import configs, ops
from tests.golden_data import load
from tests.parity import announce, assert_close_bf16, assert_close_lse

pytestmark = pytest.mark.gpu


def test_flash_forward_fixture(cuda):
    d = load("flash_forward")
    announce("golden flash_forward")
    out, lse = ops.flash_forward(d["q"].to(cuda), d["k"].to(cuda), d["v"].to(cuda), d["scale"])
    torch.cuda.synchronize()
    assert_close_bf16("O", out, d["out"])
    assert_close_lse("LSE", lse, d["lse"])


def test_mla_prefill_fixture(cuda):
    d = load("mla_prefill")
    announce("golden mla_prefill forward/backward")
    q, k, v = d["q"].to(cuda), d["k"].to(cuda), d["v"].to(cuda)
    out, lse = ops.mla_prefill_forward(q, k, v, d["scale"])
    torch.cuda.synchronize()
    assert_close_bf16("O", out, d["out"])
    assert_close_lse("LSE", lse, d["lse"])
    dq, dk, dv = ops.mla_prefill_backward(d["dout"].to(cuda), d["saved_out"].to(cuda), d["lse"].to(cuda), q, k, v,
                                          d["scale"])
    torch.cuda.synchronize()
    assert_close_bf16("dQ", dq, d["dq"])
    assert_close_bf16("dK", dk, d["dk"])
    assert_close_bf16("dV", dv, d["dv"])


def test_mla_absorbed_fixture(cuda):
    d = load("mla_absorbed")
    announce("golden mla absorbed forward/backward")
    tensors = [d[key].to(cuda) for key in ("ql", "qr", "c", "kr")]
    out, lse = ops.mla_forward(*tensors, d["scale"])
    torch.cuda.synchronize()
    assert_close_bf16("O", out, d["out"])
    assert_close_lse("LSE", lse, d["lse"])
    grads = ops.mla_backward(d["dout"].to(cuda), d["saved_out"].to(cuda), d["lse"].to(cuda), *tensors, d["scale"])
    torch.cuda.synchronize()
    for actual, key in zip(grads, ("dql", "dqr", "dc", "dkr")):
        assert_close_bf16(key, actual, d[key])


def test_mla_decode_fixture(cuda):
    d = load("mla_decode")
    announce("golden mla_decode")
    paged, table = configs.pack_cache(d["cache"], 64)
    out, lse = ops.mla_decode(d["query"].to(cuda), paged.to(cuda), table.to(cuda), d["lengths"].to(cuda), d["scale"])
    torch.cuda.synchronize()
    assert_close_bf16("O", out, d["out"])
    assert_close_lse("LSE", lse, d["lse"])

"""Who offers and who takes the norm fusion of steps with few rows, decided on the host: the
norm's row and width limits, the linear part's fallbacks, and the kernel's right to decline."""

import torch

from qwen3_from_scratch_amd import ops
from qwen3_from_scratch_amd.parts import NormSink, Precision, UnscaledRows
from qwen3_from_scratch_amd.parts.linear import LinearWeight
from qwen3_from_scratch_amd.parts.norm import RMSNorm


def _norm(size, precision):
    norm = RMSNorm("n", precision, "cpu", size=size, eps=1e-6)
    norm.weight = torch.ones(size, dtype=precision.act)
    return norm


def test_norm_offers_a_sink_by_rows_and_width():
    bf16, f32 = Precision(torch.bfloat16), Precision(torch.float32)
    stream = lambda rows, size: torch.zeros(rows, size)
    wide = _norm(128, bf16)                 # a width in steps of 64: up to 128 rows
    assert [wide.sink_for(stream(r, 128)) is not None for r in (1, 16, 17, 128, 129)] == [True, True, True, True, False]
    assert isinstance(wide.sink_for(stream(5, 128)), NormSink)
    narrow = _norm(80, bf16)                # in steps of 16 only: the few-row kernel alone
    assert [narrow.sink_for(stream(r, 80)) is not None for r in (1, 16, 17, 64)] == [True, True, False, False]
    assert _norm(72, bf16).sink_for(stream(4, 72)) is None
    assert _norm(128, f32).sink_for(stream(4, 128)) is None
    assert _norm(128, Precision(torch.bfloat16, tiled=False)).sink_for(stream(4, 128)) is None


def test_fused_rows_take_by_size():
    w = torch.zeros(256, 128, dtype=torch.bfloat16)
    assert [ops.fused_rows_take(w, m) for m in (16, 17, 128, 129)] == [False, True, True, False]
    assert not ops.fused_rows_take(torch.zeros(256, 96, dtype=torch.bfloat16), 40)       # inner size not in steps of 64
    assert not ops.fused_rows_take(torch.zeros(254, 128, dtype=torch.bfloat16), 40)      # rows of w not in steps of 4
    assert not ops.fused_rows_take(torch.zeros(256, 128), 40)                            # float32
    assert not ops.fused_rows_take(w.t(), 40)                                            # not contiguous


def test_linear_part_falls_back_where_the_kernel_declines(cpu_ops, monkeypatch):
    precision = Precision(torch.bfloat16)
    weight = (torch.randn(128, 64) * 0.1).bfloat16()
    part = LinearWeight(weight, precision)
    part.tiled = torch.zeros(1)             # the host twin keeps no tiled copy; the part only asks whether there is one
    norm = _norm(128, precision)
    x = torch.randn(40, 64).bfloat16()
    residual = torch.zeros(40, 128)
    calls = []

    def declines(x, weight, tiled, residual, norm_weight):
        calls.append(x.shape[0])
        return None

    monkeypatch.setattr(ops, "linear_residual_norm", declines, raising=False)
    out = part.forward_into(x, NormSink(residual, norm.weight, norm.eps, norm.size))
    assert calls == [40] and torch.equal(out, part.forward(x)) and float(residual.abs().max()) == 0.0

    def fuses(x, weight, tiled, residual, norm_weight):
        return torch.ones(x.shape[0], weight.shape[0], dtype=torch.bfloat16), torch.ones(1, x.shape[0])

    monkeypatch.setattr(ops, "linear_residual_norm", fuses, raising=False)
    out = part.forward_into(x, NormSink(residual, norm.weight, norm.eps, norm.size))
    assert isinstance(out, UnscaledRows) and out.width == 128 and out.sums.shape == (1, 40)
    # rows or sizes outside what the kernels take never reach them
    monkeypatch.setattr(ops, "linear_residual_norm", lambda *a: 1 / 0, raising=False)
    many = torch.randn(200, 64).bfloat16()
    assert torch.equal(part.forward_into(many, NormSink(torch.zeros(200, 128), norm.weight, norm.eps, norm.size)), part.forward(many))
    odd = LinearWeight((torch.randn(128, 96) * 0.1).bfloat16(), precision)          # inner size 96: not in steps of 64,
    odd.tiled = torch.zeros(1)                                                      # which the tiled kernel asks for
    x96 = torch.randn(100, 96).bfloat16()                                           # (more rows than the few-row kernel takes)
    assert torch.equal(odd.forward_into(x96, NormSink(torch.zeros(100, 128), norm.weight, norm.eps, norm.size)), odd.forward(x96))
    assert ops.few_rows_limit(odd.weight) == 64 and ops.few_rows_limit(torch.empty(24576, 4096, dtype=torch.bfloat16, device="meta")) == 16
    assert ops.few_rows_limit(torch.empty(8192, 1024, dtype=torch.bfloat16, device="meta")) == 32

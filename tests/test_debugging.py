"""Tracing hooks (interface of sharktank/sharktank/utils/debugging.py and layers/base.py:24-54): flag parsing, the
trace record format, golden files."""

import pytest
import torch

from sharktank_amd.utils import debugging
from sharktank_amd.layers.base import BaseLayer


@pytest.fixture
def flags():
    saved = debugging.DebugFlags(**vars(debugging.flags))
    yield debugging.flags
    for k, v in vars(saved).items():
        setattr(debugging.flags, k, v)


def test_flag_syntax():
    f = debugging.DebugFlags.parse("tensor_trace, +enable_nan_checks,save_goldens_path=/tmp/some dir/x")
    assert f.enable_tensor_trace and f.enable_nan_checks and str(f.save_goldens_path) == "/tmp/some dir/x"
    f = debugging.DebugFlags.parse("-tensor_trace,-enable_nan_checks,use_custom_iree_kernels")
    assert not f.enable_tensor_trace and not f.enable_nan_checks and f.save_goldens_path is None
    assert debugging.DebugFlags.parse("") == debugging.DebugFlags()


def test_unknown_flag_is_reported_not_fatal(capsys):
    f = debugging.DebugFlags.parse("no_such_flag,tensor_trace")
    assert f.enable_tensor_trace
    assert "no_such_flag" in capsys.readouterr().err


def test_trace_record_format(flags, capsys):
    layer = BaseLayer()
    t = torch.arange(6, dtype=torch.float16).reshape(2, 3)
    layer.trace_tensor("blk.0.out", t)
    assert capsys.readouterr().out == ""  # off by default
    flags.enable_tensor_trace = True
    layer.trace_tensor("blk.0.out", t)
    out = capsys.readouterr().out
    assert out.startswith("::: TRACE blk.0.out:default(([2, 3], torch.float16)) =\n") and "tensor(" in out
    layer.trace_tensors("blk.0", {"a": t, "b": None}, values=False)
    out = capsys.readouterr().out
    assert "blk.0:a(" in out and "...elided..." in out and "blk.0:b" not in out


def test_golden_files(flags, tmp_path, capsys):
    from safetensors.torch import load_file

    layer = BaseLayer()
    a = torch.randn(4, 5)
    layer.trace_golden("x", a)  # no path set: nothing happens
    assert list(tmp_path.iterdir()) == []
    flags.save_goldens_path = tmp_path / "g"
    flags.golden_sequence_value = 7
    layer.trace_golden("mixtral.moe_block.0.output", a)
    layer.trace_goldens("odd:key[1](2)", {"p": a.to(torch.bfloat16).t(), "q": None, "r": torch.tensor([1, 2], dtype=torch.int32)})
    names = sorted(p.name for p in (tmp_path / "g").iterdir())
    assert names == ["0007_mixtral.moe_block.0.output.safetensors", "0008_oddkey12.safetensors"]
    assert flags.golden_sequence_value == 9
    assert torch.equal(load_file(tmp_path / "g" / names[0])["default"], a)
    second = load_file(tmp_path / "g" / names[1])
    assert set(second) == {"p", "r"} and torch.equal(second["p"], a.to(torch.bfloat16).t())
    assert "::: SAVE GOLDEN" in capsys.readouterr().out
    # golden calls never print the values, traced calls never write files
    flags.enable_tensor_trace = True
    layer.trace_tensor("y", a)
    assert len(list((tmp_path / "g").iterdir())) == 2


def test_nan_check_switch(flags):
    layer = BaseLayer()
    bad = torch.tensor([1.0, float("nan")])
    layer.assert_not_nan(bad)  # off: no check
    flags.enable_nan_checks = True
    layer.assert_not_nan(torch.ones(3))
    with pytest.raises(AssertionError, match="nans"):
        layer.assert_not_nan(torch.ones(3), bad)

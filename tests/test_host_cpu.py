"""Host-side logic that needs no GPU: module plumbing and the state-dict loader."""
import pytest
import torch

from bf16_huffman_infer_amd.functional import (ANSWeight, CompressedLinear, HuffmanWeight,
                                               load_compressed_state_dict)


def _huffman_weight(M, K):
    return HuffmanWeight(
        rem=torch.zeros(1, M, K, dtype=torch.uint8), exp=torch.zeros(4096, dtype=torch.int32),
        offsets=torch.zeros(1, M, dtype=torch.int32), LUT1=torch.zeros(8192, dtype=torch.uint8),
        LUT2=torch.full((256,), 255, dtype=torch.uint8), LUT3=torch.full((256,), 255, dtype=torch.uint8),
        LUT4=torch.full((256,), 255, dtype=torch.uint8), code_lengths=torch.zeros(256, dtype=torch.uint8))


def _ans_weight(M, K):
    return ANSWeight(rem=torch.zeros(2, M, K // 2, dtype=torch.uint8), exp=torch.zeros(4096, dtype=torch.int32),
                     offsets=torch.zeros(2, M, dtype=torch.int32), LUT=torch.zeros(256, dtype=torch.int32))


def test_buffer_names_follow_the_reference_modules():
    assert [n for n, _ in _huffman_weight(128, 384).named_buffers()] == [
        "rem", "exp", "offsets", "LUT1", "LUT2", "LUT3", "LUT4", "code_lengths"]
    assert [n for n, _ in _ans_weight(128, 768).named_buffers()] == ["rem", "exp", "offsets", "LUT"]


def test_loader_rebuilds_compressed_modules_on_a_meta_skeleton():
    src = torch.nn.Sequential(
        CompressedLinear(_huffman_weight(128, 384), torch.nn.Parameter(torch.ones(128).bfloat16(), requires_grad=False)),
        torch.nn.LayerNorm(128),
        CompressedLinear(_ans_weight(256, 768), None))
    sd = src.state_dict()
    with torch.device("meta"):
        fresh = torch.nn.Sequential(torch.nn.Linear(384, 128, bias=True), torch.nn.LayerNorm(128),
                                    torch.nn.Linear(768, 256, bias=False))
    result = load_compressed_state_dict(fresh, sd)
    assert not result.missing_keys and not result.unexpected_keys
    assert type(fresh[0].weight) is HuffmanWeight and type(fresh[2].weight) is ANSWeight
    assert fresh[0].bias.device.type == "cpu" and fresh[1].weight.device.type == "cpu"
    assert fresh[2].bias is None and tuple(fresh[2].weight.rem.shape) == (2, 256, 384)


def test_loader_rejects_a_shape_mismatch():
    sd = torch.nn.Sequential(CompressedLinear(_huffman_weight(128, 384), None)).state_dict()
    with pytest.raises(RuntimeError, match="expects"):
        load_compressed_state_dict(torch.nn.Sequential(torch.nn.Linear(512, 128, bias=False)), sd)


def test_compressed_ops_refuse_cpu_tensors():
    w = _huffman_weight(128, 384)
    with pytest.raises((AssertionError, RuntimeError, NotImplementedError)):
        torch.nn.functional.linear(torch.zeros(1, 384, dtype=torch.bfloat16), w)


def test_missing_library_is_a_loud_error(monkeypatch, tmp_path):
    """There is no fallback: without the built HIP library nothing of the package runs."""
    from bf16_huffman_infer_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libbhi_hip.so"))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        _lib.load()
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        _lib.constants()


def test_package_does_not_import_the_oracle():
    import subprocess
    import sys
    code = ("import sys, bf16_huffman_infer_amd, bf16_huffman_infer_amd.cudagraph_utils, "
            "bf16_huffman_infer_amd.reference_format; "
            "assert not [m for m in sys.modules if m == 'oracle' or m.startswith('oracle.')]")
    subprocess.run([sys.executable, "-c", code], check=True, cwd=__import__("os").path.dirname(
        __import__("os").path.dirname(__import__("os").path.abspath(__file__))))


def test_bench_refuses_more_than_one_gpu():
    """This build measures one GPU; asking the benchmark for more must say so and stop."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=300)
    assert r.returncode != 0
    assert "one GPU" in (r.stderr + r.stdout)

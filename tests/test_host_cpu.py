"""Host-side logic that needs no GPU: module plumbing and the state-dict loader."""
import pytest
import torch

from bf16_huffman_infer_amd.functional import (ANSWeight, CompressedLinear, HuffmanWeight,
                                               load_compressed_state_dict)


def _task_offsets(split_k, M, words_per_task=64):
    """offsets of a stream with one chunk per row group and equally long tasks (the shapes
    used here have three steps per split, hence a single chunk)."""
    off = torch.zeros(split_k, M // 4, 4, dtype=torch.int32)
    off[:, :, 0] = (torch.arange(split_k * (M // 4), dtype=torch.int32) * words_per_task).view(split_k, M // 4)
    return off.view(split_k, M), split_k * (M // 4) * words_per_task + 2048


def _huffman_weight(M, K, header=(2, 11, 11, 0)):
    offsets, words = _task_offsets(1, M)
    code_lengths = torch.zeros(256, dtype=torch.uint8)
    code_lengths[:4] = torch.tensor(header, dtype=torch.uint8)
    return HuffmanWeight(
        rem=torch.zeros(1, M, K, dtype=torch.uint8), exp=torch.zeros(words, dtype=torch.int32),
        offsets=offsets, LUT1=torch.zeros(8192, dtype=torch.uint8),
        LUT2=torch.full((256,), 255, dtype=torch.uint8), LUT3=torch.full((256,), 255, dtype=torch.uint8),
        LUT4=torch.full((256,), 255, dtype=torch.uint8), code_lengths=code_lengths)


def _ans_weight(M, K):
    offsets, words = _task_offsets(2, M)
    return ANSWeight(rem=torch.zeros(2, M, K // 2, dtype=torch.uint8), exp=torch.zeros(words, dtype=torch.int32),
                     offsets=offsets, LUT=torch.zeros(256, dtype=torch.int32))


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


def test_gemm_workspace_is_keyed_by_device_and_stream():
    """Two streams must get two workspaces (launches on them may overlap); one stream keeps its
    own, which grows by replacement while the old one stays alive for launches still enqueued."""
    from bf16_huffman_infer_amd import ops
    cpu = torch.device("cpu")
    make = lambda n: torch.zeros(n, dtype=torch.uint8)
    saved = dict(ops._workspaces)
    ops._workspaces.clear()
    try:
        a = ops._gemm_workspace(cpu, 11, 100, allocate=make)
        b = ops._gemm_workspace(cpu, 22, 100, allocate=make)
        assert a.data_ptr() != b.data_ptr()
        assert ops._gemm_workspace(cpu, 11, 50, allocate=make) is a
        big = ops._gemm_workspace(cpu, 11, 4 << 20, allocate=make)
        assert big is not a and big.numel() >= 4 << 20 and not bool(big.any())
        assert any(t is a for t in ops._workspaces[(cpu, 11)]), "the smaller workspace must stay alive"
        assert ops._gemm_workspace(cpu, 22, 100, allocate=make) is b
    finally:
        ops._workspaces.clear()
        ops._workspaces.update(saved)


def test_dispatch_rule_between_gemv_and_matrix_cores():
    """The measured rule: small layers and few rows stay on the GEMV; long-K and large layers move to
    the matrix-core kernel from 4, 6 or 8 rows."""
    from bf16_huffman_infer_amd.functional import prefers_matrix_cores
    for M, K in ((4608, 3584), (3584, 3584), (4096, 4096), (1024, 4096), (6144, 4096), (8192, 8192)):
        assert not any(prefers_matrix_cores(r, M, K) for r in range(1, 9)), (M, K)
    want = {(3584, 18944): [4, 5, 6, 7, 8], (14336, 4096): [4, 5, 6, 7, 8], (18944, 3584): [6, 7, 8],
            (12288, 4096): [6, 7, 8], (11008, 4096): [6, 7, 8], (4096, 14336): [6, 7, 8],
            (4096, 12288): [8], (4096, 11008): [8], (37888, 3584): [3, 4, 5, 6, 7, 8], (152064, 3584): [3, 4, 5, 6, 7, 8]}
    for (M, K), rows in want.items():
        assert [r for r in range(1, 9) if prefers_matrix_cores(r, M, K)] == rows, (M, K)


def test_binding_checks_the_member_struct_against_the_library():
    import ctypes
    from bf16_huffman_infer_amd import _lib
    assert _lib.constants()["member_bytes"] == ctypes.sizeof(_lib.GemvMember) == 88


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


def _ans_buffers(layout: str, M=128, K=512):
    """(rem, exp, offsets, LUT) of a seeded matrix in this package's layout ('wave64') or in the
    reference package's ('reference'), both written by the numpy models."""
    import numpy as np
    from helpers import bits_of, gaussian_weight
    from oracle import planes, ref_layout, ref_tables, wave64
    bits = bits_of(gaussian_weight(M, K, seed=2))
    _, exp = planes.split_bf16(bits)
    freq, cum, lut = ref_tables.ans_tables(np.bincount(exp.reshape(-1), minlength=256))
    enc = (wave64.encode_ans(bits, 1, np.asarray(freq), np.asarray(cum)) if layout == "wave64"
           else ref_layout.encode(bits, 1, "ans", (np.asarray(freq), np.asarray(cum))))
    return (torch.from_numpy(enc["rem"].copy()), torch.from_numpy(enc["exp"].copy()),
            torch.from_numpy(enc["offsets"].copy()), torch.from_numpy(np.asarray(lut, dtype=np.int32)))


def test_layout_check_accepts_this_packages_buffers_and_rejects_the_references():
    """A rANS weight saved by the reference package has the same names, dtypes and shapes; only
    its contents tell it apart, and the kernels must never see it."""
    from bf16_huffman_infer_amd.functional import check_layout
    check_layout(ANSWeight(*_ans_buffers("wave64")))
    with pytest.raises(RuntimeError, match="transcode_reference_weight"):
        check_layout(ANSWeight(*_ans_buffers("reference")))
    sd = torch.nn.Sequential(CompressedLinear(ANSWeight(*_ans_buffers("reference")), None)).state_dict()
    with pytest.raises(RuntimeError, match="transcode_reference_weight"):
        load_compressed_state_dict(torch.nn.Sequential(torch.nn.Linear(512, 128, bias=False)), sd)


def test_layout_check_reads_the_huffman_header():
    from bf16_huffman_infer_amd.functional import check_layout
    w = _huffman_weight(128, 384, header=(0, 0, 0, 0))        # not this package's format version
    with pytest.raises(RuntimeError, match="Huffman tables"):
        check_layout(w)


def test_nibble_window_leaves_room_for_the_escape_nibble():
    """base + 15 must fit a byte (the decoder adds the base to four nibbles in one 32-bit add)."""
    from bf16_huffman_infer_amd.functional import NibbleCodec
    counts = torch.zeros(256, dtype=torch.int64)
    counts[241:256] = 1000                        # the densest 15-wide window starts at 241
    counts[3] = 1
    codec = NibbleCodec(counts)
    assert codec.base == 240 and codec.has_escapes


def test_single_split_weights_may_omit_the_split_dimension():
    """mv_huffman / mv_ans accept rem [M, N] with offsets [M] (reference functional.py:33-36)."""
    from bf16_huffman_infer_amd.functional import _promote_single_split
    rem, off = _promote_single_split(torch.zeros(128, 384, dtype=torch.uint8), torch.zeros(128, dtype=torch.int32))
    assert tuple(rem.shape) == (1, 128, 384) and tuple(off.shape) == (1, 128)
    rem3, off2 = torch.zeros(2, 128, 384, dtype=torch.uint8), torch.zeros(2, 128, dtype=torch.int32)
    assert _promote_single_split(rem3, off2)[0] is rem3 and _promote_single_split(rem3, off2)[1] is off2


def test_get_model_size_counts_parameters_and_buffers():
    from bf16_huffman_infer_amd.utils import get_model_size
    lin = CompressedLinear(_huffman_weight(128, 384), torch.nn.Parameter(torch.ones(128).bfloat16(), requires_grad=False))
    want = sum(b.nelement() * b.element_size() for b in lin.weight.buffers()) + 128 * 2
    assert get_model_size(lin) == want == 128 * 384 + (32 * 64 + 2048) * 4 + 128 * 4 + 8192 + 4 * 256 + 256


def test_workspace_of_the_fused_product_follows_the_slice_choice():
    """`bhi_gemm_workspace_bytes` is host arithmetic: 1 KiB of arrival counters plus
    slices x rows x M floats, nothing for a weight that is not cut along K.  The slice counts
    are the ones measured fastest on the GPU for these shapes."""
    from bf16_huffman_infer_amd import _lib
    lib = _lib.load()

    def slices(split_k, M, Ks, rows):
        need = lib.bhi_gemm_workspace_bytes(split_k, M, Ks, rows)
        if need == 0:
            return 1
        assert (need - 1024) % (rows * M * 4) == 0
        return (need - 1024) // (rows * M * 4)

    assert slices(1, 12288, 4096, 16) == 1 and slices(1, 12288, 4096, 32) == 1      # 3072 row groups: never cut
    assert slices(3, 4096, 4096, 16) == 4 and slices(3, 4096, 4096, 32) == 4        # 4096x12288, 12 tasks per group
    assert slices(4, 3584, 4736, 16) == 4 and slices(4, 3584, 4736, 32) == 4        # 3584x18944, 4 long tasks
    assert slices(1, 4096, 4096, 16) == 2 and slices(1, 4608, 3584, 16) == 2
    # every choice divides the tasks of a row group, and the built-in workspace holds whatever
    # stays within one block per compute unit
    static = lib.bhi_gemm_static_workspace_bytes()
    for split_k, M, Ks in [(1, 1024, 4096), (2, 2048, 2048), (8, 4096, 1024), (3, 4096, 4096), (1, 8128, 3584)]:
        per_group = split_k * lib.bhi_chunks_per_group(M, Ks, split_k)
        for rows in (9, 16, 17, 32):
            d = slices(split_k, M, Ks, rows)
            assert per_group % d == 0
            if (M // 4 // (8 if rows <= 16 else 16)) * d <= 256:
                assert lib.bhi_gemm_workspace_bytes(split_k, M, Ks, rows) <= static

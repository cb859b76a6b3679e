"""Buffers in the reference's own layout (built by the numpy restatement of its encoder,
with tables written by its own table builder) are read back by the HIP reader."""
import json
import os

import numpy as np
import pytest
import torch

from helpers import bits_of, gaussian_weight, student_t_weight

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _t(a):
    return torch.from_numpy(np.ascontiguousarray(a))


@pytest.mark.parametrize("name,split_k", [("gaussian_exponents", 1), ("student_t_exponents", 2), ("powers_of_two_30", 1)])
def test_reference_huffman_buffers_decode_and_transcode(cuda, name, split_k):
    from bf16_huffman_infer_amd.reference_format import decode_reference_huffman, transcode_reference_weight
    from oracle import ref_layout
    with open(os.path.join(GOLDEN, "huffman_tables.json")) as f:
        v = json.load(f)[name]
    luts = np.array([v["LUT1"], v["LUT2"], v["LUT3"], v["LUT4"]], dtype=np.uint8)
    lens = np.array(v["code_lengths"], dtype=np.uint8)
    codes = {int(s): (int(c, 2), len(c)) for s, c in v["codes"].items()}
    counts = np.asarray(v["counts"], dtype=np.float64)
    rng = np.random.default_rng(5)
    M, K = 256, 768
    exp = rng.choice(256, size=(M, K), p=counts / counts.sum()).astype(np.uint16)
    rem = rng.integers(0, 256, size=(M, K)).astype(np.uint16)
    bits = (((rem << 8) & 0x8000) | (rem & 0x7F) | (exp << 7)).astype(np.uint16)
    enc = ref_layout.encode(bits, split_k, "huffman", codes)
    buffers = dict(rem=_t(enc["rem"]), exp=_t(enc["exp"]), offsets=_t(enc["offsets"]),
                   LUT1=_t(luts[0]), LUT2=_t(luts[1]), LUT3=_t(luts[2]), LUT4=_t(luts[3]), code_lengths=_t(lens))
    got = decode_reference_huffman(**buffers)
    assert np.array_equal(got.cpu().view(torch.int16).numpy().view(np.uint16), bits)
    if name != "powers_of_two_30":           # a 30-level histogram is not compressible enough to be interesting
        mine = transcode_reference_weight(buffers).cuda()
        assert type(mine).__name__ == "HuffmanWeight"
        assert np.array_equal(mine.get_weight().cpu().view(torch.int16).numpy().view(np.uint16), bits)


@pytest.mark.parametrize("maker,split_k", [(gaussian_weight, 1), (student_t_weight, 3)])
def test_reference_ans_buffers_decode_and_transcode(cuda, maker, split_k):
    from bf16_huffman_infer_amd.reference_format import decode_reference_ans, transcode_reference_weight
    from oracle import planes, ref_layout, ref_tables
    w = maker(128, 384 * split_k, seed=8)
    bits = bits_of(w)
    _, exp = planes.split_bf16(bits)
    freq, cum, lut = ref_tables.ans_tables(np.bincount(exp.reshape(-1), minlength=256), 8)
    enc = ref_layout.encode(bits, split_k, "ans", (freq, cum))
    buffers = dict(rem=_t(enc["rem"]), exp=_t(enc["exp"]), offsets=_t(enc["offsets"]), LUT=_t(lut))
    got = decode_reference_ans(**buffers)
    assert np.array_equal(got.cpu().view(torch.int16).numpy().view(np.uint16), bits)
    mine = transcode_reference_weight(buffers, algo="smallest").cuda()
    assert torch.equal(mine.get_weight().cpu().view(torch.int16), w.view(torch.int16))


@pytest.mark.parametrize("algo", ["huffman", "ans"])
@pytest.mark.parametrize("K,split_k", [(384, 1), (768, 2)])
def test_reference_buffers_of_several_parts(cuda, K, split_k, algo):
    """8320 rows: three 4096-row parts per split, each followed by its 64 zero words, offsets
    running on across parts and splits (reference ``functional.py:202-231``) -- the shape of
    every layer of a real checkpoint."""
    from bf16_huffman_infer_amd.reference_format import (decode_reference_ans, decode_reference_huffman,
                                                         transcode_reference_weight)
    from test_oracle_cpu import multi_part_case
    bits, enc, tables, _ = multi_part_case(K, split_k, algo)
    buffers = dict(rem=_t(enc["rem"]), exp=_t(enc["exp"]), offsets=_t(enc["offsets"]))
    if algo == "huffman":
        luts, lens = tables
        buffers.update(LUT1=_t(luts[0]), LUT2=_t(luts[1]), LUT3=_t(luts[2]), LUT4=_t(luts[3]), code_lengths=_t(lens))
        got = decode_reference_huffman(**buffers)
    else:
        buffers.update(LUT=_t(tables[0]))
        got = decode_reference_ans(**buffers)
    assert np.array_equal(got.cpu().view(torch.int16).numpy().view(np.uint16), bits)
    mine = transcode_reference_weight(buffers).cuda()
    assert type(mine).__name__ == ("HuffmanWeight" if algo == "huffman" else "ANSWeight")
    assert np.array_equal(mine.get_weight().cpu().view(torch.int16).numpy().view(np.uint16), bits)

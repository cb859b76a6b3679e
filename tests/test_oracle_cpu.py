"""CPU checks that pin the oracle and the host-side logic (no GPU needed)."""
import numpy as np
import pytest
import torch

from helpers import (bits_of, gaussian_weight, pair_counts, random_bits_weight, special_values_weight,
                     student_t_weight)
from oracle import planes, ref_layout, ref_tables, wave64


# ----------------------------------------------------------------------------- bit planes
def test_split_rebuild_all_65536_patterns():
    bits = np.arange(65536, dtype=np.uint16)
    rem, exp = planes.split_bf16(bits)
    assert np.array_equal(planes.rebuild_bf16(rem, exp), bits)
    # field positions against IEEE bfloat16: sign 15, exponent 14..7, mantissa 6..0
    f = torch.from_numpy(bits.view(np.int16)).view(torch.bfloat16).float()
    m, e = torch.frexp(f[(exp > 0) & (exp < 255)])
    assert np.array_equal((e.numpy() + 126).astype(np.uint8), exp[(exp > 0) & (exp < 255)])
    assert np.array_equal((rem >> 7).astype(bool), (bits >> 15).astype(bool))
    assert np.array_equal(rem & 0x7F, (bits & 0x7F).astype(np.uint8))


def test_product_split_matches_oracle():
    from bf16_huffman_infer_amd.utils import split_bf16
    w = special_values_weight(64, 128, seed=2)
    rem, exp = split_bf16(w)
    orem, oexp = planes.split_bf16(bits_of(w))
    assert np.array_equal(rem.numpy(), orem) and np.array_equal(exp.numpy(), oexp)


@pytest.mark.parametrize("n,want", [(4096, 1), (3584, 1), (12288, 3), (18944, 4), (11008, 2), (384, 1),
                                    (8192, 2), (5120, 2), (14336, 4), (28672, 7)])
def test_block_size_table(n, want):
    from bf16_huffman_infer_amd.utils import get_block_size_n
    assert planes.get_block_size_n(n) == want
    assert get_block_size_n(torch.empty(1, n)) == (want,)


@pytest.mark.parametrize("n", [128, 256, 100, 4097])
def test_block_size_rejects(n):
    from bf16_huffman_infer_amd.utils import get_block_size_n
    with pytest.raises(RuntimeError):
        planes.get_block_size_n(n)
    with pytest.raises(RuntimeError):
        get_block_size_n(torch.empty(1, n))


# ----------------------------------------------------------------------------- reference tables
def test_ans_tables_worked_example():
    sample = [1, 2, 3, 3, 2, 12, 13, 11, 1, 8, 1, 7, 1, 6, 1, 1]
    freq, cum, lut = ref_tables.ans_tables(np.bincount(sample, minlength=256))
    assert {s: int(f) for s, f in enumerate(freq) if f} == {1: 96, 2: 32, 3: 32, 6: 16, 7: 16, 8: 16, 11: 16,
                                                            12: 16, 13: 16}
    assert {s: int(cum[s]) for s in range(256) if freq[s]} == {1: 0, 2: 96, 3: 128, 6: 160, 7: 176, 8: 192,
                                                               11: 208, 12: 224, 13: 240}
    words, n = ref_layout._ans_words(np.array([[1]], dtype=np.uint8), freq, cum)
    assert n[0] == 1 and words[0, 0] == 576            # 256/96 -> q=2, r=64 -> (2<<8)+64
    e = int(lut.view(np.uint32)[576 & 255])
    assert (e >> 24, (e >> 12) & 0xFFF, e & 0xFFF) == (1, 96, 64)
    assert 96 * (576 >> 8) + 64 == 256


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_ans_tables_invariants_and_product_agreement(seed):
    from bf16_huffman_infer_amd.ans import RANSEncoder
    rng = np.random.default_rng(seed)
    counts = np.zeros(256, dtype=np.int64)
    syms = rng.choice(256, size=40, replace=False)
    counts[syms] = (rng.pareto(0.7, size=40) * 50 + 1).astype(np.int64)
    freq, cum, lut = ref_tables.ans_tables(counts)
    assert freq.sum() == 256 and ((freq > 0) == (counts > 0)).all()
    assert np.array_equal(cum, np.cumsum(freq) - freq)
    u = lut.view(np.uint32)
    for slot in range(256):
        s, f, r = int(u[slot] >> 24), int((u[slot] >> 12) & 0xFFF), int(u[slot] & 0xFFF)
        assert f == freq[s] and slot == cum[s] + r
    codec = RANSEncoder(counts.tolist(), precision=8)
    assert codec.freq == freq.tolist() and codec.cum == cum.tolist()
    packed = [(s << 24) | (f << 12) | r for s, f, r in codec.decode_lut]
    assert packed == u.tolist()


@pytest.mark.parametrize("maker", [gaussian_weight, student_t_weight])
def test_cascade_tables_decode_every_code(maker):
    _, exp = planes.split_bf16(bits_of(maker(256, 1024, seed=4)))
    counts = np.bincount(exp.reshape(-1), minlength=256)
    luts, lens, codes = ref_tables.build_cascade_luts(counts)
    kraft = sum(2.0 ** -l for _, l in codes.values())
    assert abs(kraft - 1.0) < 1e-12 and max(l for _, l in codes.values()) <= 32
    for s, (code, ln) in codes.items():
        for junk in (0, 0xFFFFFFFF, 0x5A5A5A5A):
            window = (code | (junk << ln)) & 0xFFFFFFFF
            assert ref_tables.decode_code(luts, lens, window) == (s, ln)
    p = counts[counts > 0] / counts.sum()
    avg = sum(counts[s] * l for s, (_, l) in codes.items()) / counts.sum()
    assert -(p * np.log2(p)).sum() <= avg < -(p * np.log2(p)).sum() + 1


def test_reference_layout_index_facts():
    idx = np.arange(256, dtype=np.uint8)[None, :]
    so = ref_layout.stream_order(idx)
    assert so[0, 0].tolist() == [0, 1, 128, 129] and so[0, 33].tolist() == [66, 67, 194, 195]
    assert np.array_equal(ref_layout.stream_order_inverse(so), idx)
    pr = ref_layout.permute_rem(np.arange(128, dtype=np.uint8)[None, :])
    assert pr[0, :4].tolist() == [0, 1, 64, 65]
    assert np.array_equal(ref_layout.permute_rem_inverse(pr), np.arange(128, dtype=np.uint8)[None, :])


@pytest.mark.parametrize("maker,M,K,split_k", [(gaussian_weight, 128, 512, 1), (student_t_weight, 256, 1024, 2)])
def test_reference_layout_round_trip(maker, M, K, split_k):
    bits = bits_of(maker(M, K, seed=6))
    _, exp = planes.split_bf16(bits)
    counts = np.bincount(exp.reshape(-1), minlength=256)
    luts, lens, codes = ref_tables.build_cascade_luts(counts)
    enc = ref_layout.encode(bits, split_k, "huffman", codes)
    assert enc["rem"].shape == (split_k, M, K // split_k) and enc["offsets"].shape == (split_k, M)
    assert np.array_equal(ref_layout.decode_huffman(enc["rem"], enc["exp"], enc["offsets"], luts, lens), bits)
    freq, cum, lut = ref_tables.ans_tables(counts)
    enc = ref_layout.encode(bits, split_k, "ans", (freq, cum))
    assert np.array_equal(ref_layout.decode_ans(enc["rem"], enc["exp"], enc["offsets"], lut), bits)


def multi_part_case(K, split_k, algo, seed=6):
    """8320 rows = two whole parts of 4096 and one of 128, as every layer of a real model has
    (reference ``functional.py:202-209``).  Returns (bits, encoded buffers, decode tables)."""
    bits = bits_of(gaussian_weight(8320, K, seed=seed))
    _, exp = planes.split_bf16(bits)
    counts = np.bincount(exp.reshape(-1), minlength=256)
    if algo == "huffman":
        luts, lens, codes = ref_tables.build_cascade_luts(counts)
        return bits, ref_layout.encode(bits, split_k, "huffman", codes), (luts, lens), codes
    freq, cum, lut = ref_tables.ans_tables(counts)
    return bits, ref_layout.encode(bits, split_k, "ans", (freq, cum)), (lut,), (freq, cum)


@pytest.mark.parametrize("algo", ["huffman", "ans"])
@pytest.mark.parametrize("K,split_k", [(384, 1), (768, 1), (768, 2)])
def test_reference_layout_parts_pads_and_rebased_offsets(K, split_k, algo):
    """Several 4096-row parts per split: 64 zero words behind every part (reference
    ``functional.py:177``), offsets running on across parts and splits (``:210-231``), and a part's
    words independent of what surrounds it."""
    bits, enc, tables, enc_tables = multi_part_case(K, split_k, algo)
    M, Ks = bits.shape[0], K // split_k
    exp, off = enc["exp"].view(np.uint32), enc["offsets"].astype(np.int64)
    part_starts = [0, 4096, 8192]
    assert off[0, 0] == 0 and (np.diff(off.reshape(-1)) > 0).all()
    ends = np.append(off.reshape(-1)[1:], exp.size)                  # where the next row (or the stream) begins
    for k in range(split_k):
        for j, r0 in enumerate(part_starts):
            r1 = min(r0 + 4096, M)
            # the part's rows are followed by exactly one row of 64 zero words, which belongs to no row
            part_end = ends[k * M + r1 - 1]
            assert not exp[part_end - 64:part_end].any()
            row_words = np.diff(np.append(off[k, r0:r1], part_end - 64))
            assert (row_words % 64 == 0).all() and (row_words > 0).all()
            # the same rows compressed on their own: the same words, offsets shifted by the part's base
            alone = ref_layout.encode(bits[r0:r1, k * Ks:(k + 1) * Ks], 1, algo, enc_tables)
            assert np.array_equal(alone["exp"].view(np.uint32), exp[off[k, r0]:part_end])
            assert np.array_equal(alone["offsets"][0].astype(np.int64) + off[k, r0], off[k, r0:r1])
    assert ends[-1] == exp.size
    if algo == "huffman":
        got = ref_layout.decode_huffman(enc["rem"], enc["exp"], enc["offsets"], *tables)
    else:
        got = ref_layout.decode_ans(enc["rem"], enc["exp"], enc["offsets"], *tables)
    assert np.array_equal(got, bits)


def test_reference_cascade_hole_is_real():
    """The reference reserves 255 as the miss marker, so exponent 255 (inf/NaN) cannot be
    told from a miss; recorded here so nobody trusts the cascade on such tensors."""
    counts = np.zeros(256, dtype=np.int64)
    counts[[120, 121, 255]] = [1000, 900, 50]
    luts, lens, codes = ref_tables.build_cascade_luts(counts)
    code, ln = codes[255]
    with pytest.raises(AssertionError):
        assert ref_tables.decode_code(luts, lens, code) == (255, ln)


# ----------------------------------------------------------------------------- wave64 format
def _codec(bits):
    from bf16_huffman_infer_amd.huffman import LUTHuffmanEncoder
    codec = LUTHuffmanEncoder()
    codec.build_lut(pair_counts(bits))
    wave64.check_tables(codec.dec_table, codec.enc_table)
    return codec


@pytest.mark.parametrize("maker,M,K,split_k", [
    (gaussian_weight, 128, 384, 1), (gaussian_weight, 256, 512, 2), (student_t_weight, 128, 1024, 1),
    (random_bits_weight, 128, 384, 1), (special_values_weight, 128, 640, 1),
    (lambda M, K, seed: torch.zeros(M, K, dtype=torch.bfloat16), 128, 128, 1),
    (gaussian_weight, 1024, 2048, 1),
])
def test_wave64_round_trip(maker, M, K, split_k):
    bits = bits_of(maker(M, K, seed=9))
    codec = _codec(bits)
    enc = wave64.encode(bits, split_k, codec.enc_table)
    assert enc["rem"].shape == (split_k, M, K // split_k) and enc["offsets"].shape == (split_k, M)
    assert len(enc["exp"]) % wave64.ALIGN_WORDS == 0
    assert np.array_equal(wave64.decode(enc["rem"], enc["exp"], enc["offsets"], codec.dec_table), bits)


def test_wave64_and_reference_layout_agree():
    bits = bits_of(gaussian_weight(128, 768, seed=12))
    codec = _codec(bits)
    a = wave64.encode(bits, 1, codec.enc_table)
    _, exp = planes.split_bf16(bits)
    luts, lens, codes = ref_tables.build_cascade_luts(np.bincount(exp.reshape(-1), minlength=256))
    b = ref_layout.encode(bits, 1, "huffman", codes)
    da = wave64.decode(a["rem"], a["exp"], a["offsets"], codec.dec_table)
    db = ref_layout.decode_huffman(b["rem"], b["exp"], b["offsets"], luts, lens)
    assert np.array_equal(da, db) and np.array_equal(da, bits)
    # the shared-stream layout has no per-row padding: it must not be larger
    assert a["exp"].nbytes - 4 * wave64.TAIL_PAD_WORDS < b["exp"].nbytes


def test_wave64_escape_list_and_cursor_edges():
    """Hand-made code: three coded pairs and ESC; rows alternate so that every lane meets
    escapes, 1-bit codes and longest codes, and cursors cross words at different steps."""
    enc = np.zeros(wave64.ESC_INDEX + 1, dtype=np.uint32)
    dec = np.zeros(1 << wave64.TABLE_BITS, dtype=np.uint32)
    TB = wave64.TABLE_BITS
    table = {0x7878: (0b0, 1), 0x7979: (0b01, 2), 0x7A7A: ((1 << TB) - 5, TB), wave64.ESC_INDEX: ((1 << (TB - 1)) - 5, TB)}
    for p, (code, ln) in table.items():
        enc[p] = code | (ln << 16)
    # complete the code with filler pairs so that every table index resolves
    filler = 0x0101
    used = np.zeros(1 << TB, dtype=bool)
    for p, (code, ln) in table.items():
        idx = code + (np.arange(1 << (TB - ln)) << ln)
        used[idx] = True
    # every unused index becomes its own longest code of a filler pair
    for idx in np.nonzero(~used)[0]:
        enc[filler] = int(idx) | (TB << 16)
        table[filler] = (int(idx), TB)
        filler += 1
    for p, (code, ln) in table.items():
        idx = code + (np.arange(1 << (TB - ln)) << ln)
        dec[idx] = (ln | wave64.ESC_FLAG) if p == wave64.ESC_INDEX else (ln | ((p & 0xFF) << 7) | ((p >> 8) << 23))
    wave64.check_tables(dec, enc)
    rng = np.random.default_rng(0)
    M, K = 128, 1536
    choices = np.array([0x7878, 0x7979, 0x7A7A, 0x1234, 0xFFFE], dtype=np.uint16)   # last two are escaped
    pr = choices[rng.choice(5, size=(M, K // 2), p=[0.55, 0.2, 0.1, 0.1, 0.05])]
    exp = np.stack([pr & 0xFF, pr >> 8], axis=-1).reshape(M, K).astype(np.uint16)
    bits = ((exp << 7) | rng.integers(0, 128, size=(M, K)).astype(np.uint16)
            | (rng.integers(0, 2, size=(M, K)).astype(np.uint16) << 15)).astype(np.uint16)
    out = wave64.encode(bits, 1, enc)
    assert np.array_equal(wave64.decode(out["rem"], out["exp"], out["offsets"], dec), bits)


def test_chunk_rule_matches_library():
    from bf16_huffman_infer_amd import _lib
    lib = _lib.load()
    for M, Ks, sk in [(4096, 4096, 1), (4608, 3584, 1), (3584, 3584, 1), (18944, 3584, 1), (3584, 4736, 4),
                      (12288, 4096, 1), (4096, 4096, 3), (128, 384, 1), (151936, 4096, 1), (1024, 4096, 1)]:
        assert lib.bhi_chunks_per_group(M, Ks, sk) == wave64.chunks_per_group(M, Ks, sk)
    c = _lib.constants()
    assert (c["lanes"], c["group_rows"], c["step_cols"], c["table_bits"], c["window_words"], c["header_bits"],
            c["align_words"], c["tail_pad_words"], c["target_tasks"]) == (
        wave64.LANES, wave64.GROUP_ROWS, wave64.STEP_COLS, wave64.TABLE_BITS, wave64.WINDOW_WORDS,
        wave64.HEADER_BITS, wave64.ALIGN_WORDS, wave64.TAIL_PAD_WORDS, wave64.TARGET_TASKS)


# ----------------------------------------------------------------------------- pair code builder
def test_package_merge_is_optimal_on_small_alphabets():
    """Brute force over all length assignments with Kraft sum <= 1."""
    from itertools import product
    from bf16_huffman_infer_amd.huffman import package_merge
    rng = np.random.default_rng(3)
    for n, L in [(3, 2), (4, 3), (5, 3), (6, 3), (5, 4)]:
        for _ in range(20):
            w = [int(x) for x in rng.integers(1, 100, size=n)]
            got = package_merge(w, L)
            assert max(got) <= L and sum(2.0 ** -l for l in got) <= 1 + 1e-12
            best = min(sum(a * b for a, b in zip(w, ls)) for ls in product(range(1, L + 1), repeat=n)
                       if sum(2.0 ** -l for l in ls) <= 1 + 1e-12)
            assert sum(a * b for a, b in zip(w, got)) == best


def test_pair_code_beats_entropy_bound_plus_margin():
    bits = bits_of(gaussian_weight(1024, 1024, seed=21))
    counts = pair_counts(bits)
    codec = _codec(bits)
    p = counts[counts > 0] / counts.sum()
    h_pair = -(p * np.log2(p)).sum()
    avg = codec.expected_bits / counts.sum()
    assert h_pair <= avg < h_pair + 0.2
    assert (codec.enc_table >> 16).max() <= 12


def test_c_abi_exports_every_declared_symbol():
    import ctypes
    import os
    import re
    from bf16_huffman_infer_amd import _lib
    header = open(os.path.join(os.path.dirname(__file__), "..", "include", "bhi.h")).read()
    declared = set(re.findall(r"\b(bhi_[a-z0-9_]+)\s*\(", header))
    assert declared == set(_lib.EXPORTS)
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), name
    # the one struct of the ABI: the header states its size, the library asserts it at compile time
    assert ctypes.sizeof(_lib.GemvMember) == 88 and "88 bytes" in header
    assert [f[0] for f in _lib.GemvMember._fields_] == re.findall(
        r"^\s+(?:const )?(?:void\*|int64_t|int32_t) (\w+);", header[header.index("typedef struct bhi_gemv_member"):], re.M)


# ----------------------------------------------------------------------------- rANS in the wave64 layout

@pytest.mark.parametrize("kind,M,K,n", [("gauss", 64, 1024, 1), ("t3", 32, 768, 2), ("bits", 16, 384, 1),
                                        ("special", 32, 512, 1), ("zeros", 8, 384, 1)])
def test_wave64_ans_round_trip(kind, M, K, n):
    makers = {"gauss": gaussian_weight, "t3": student_t_weight, "bits": random_bits_weight,
              "special": special_values_weight, "zeros": lambda M, K, seed=0: torch.zeros(M, K, dtype=torch.bfloat16)}
    bits = bits_of(makers[kind](M, K, seed=2))
    _, exp = planes.split_bf16(bits)
    freq, cum, lut = ref_tables.ans_tables(np.bincount(exp.reshape(-1), minlength=256), 8)
    enc = wave64.encode_ans(bits, n, freq, cum)
    assert enc["exp"].dtype == np.int32 and (len(enc["exp"]) - wave64.TAIL_PAD_WORDS) % wave64.ALIGN_WORDS == 0
    assert np.array_equal(wave64.decode_ans(enc["rem"], enc["exp"], enc["offsets"], lut), bits)
    # the reference layout with the reference's own schedule gives back the same tensor
    ref = ref_layout.encode(bits, n, "ans", (freq, cum))
    assert np.array_equal(ref_layout.decode_ans(ref["rem"], ref["exp"], ref["offsets"], lut), bits)


def test_wave64_ans_state_schedule_by_hand():
    """One lane worked by hand with the tables of ans.py:152 (freq 1:96 2:32 3:32 ...).

    Symbols of the only step: [1,1,1,1 | 1,1,1,1].  Encoder, backwards from x = 2**32:
    second half: x >= 2**32 and fits -> no word; four pushes of symbol 1 (f=96, c=0):
    x -> ((x // 96) << 8) + x % 96, four times; first half: same.  The block then holds
    the final state in rows 1 (high word) and 0 (low word), and the decoder must come
    back to exactly 2**32 without ever pulling a word."""
    counts = np.bincount([1, 2, 3, 3, 2, 12, 13, 11, 1, 8, 1, 7, 1, 6, 1, 1], minlength=256)
    freq, cum, lut = ref_tables.ans_tables(counts, 8)
    x = 1 << 32
    for _ in range(8):
        x = ((x // 96) << 8) + x % 96
    sym = np.ones((1, 1, wave64.LANES, wave64.LANE_COLS), dtype=np.uint8)
    blk = wave64._ans_encode_tasks(sym, freq, cum)[0]
    assert len(blk) == 2 * wave64.LANES
    assert (blk[:wave64.LANES] == (x & 0xFFFFFFFF)).all() and (blk[wave64.LANES:] == (x >> 32)).all()
    words = np.concatenate([blk, np.zeros(256, dtype=np.uint32)])
    out = wave64._ans_decode_tasks(words, np.array([0]), 1, lut.view(np.uint32))
    assert (out == 1).all()


def test_ans_capacity_matches_library():
    from bf16_huffman_infer_amd import _lib
    lib = _lib.load()
    for ns in (1, 4, 28, 37, 128):
        assert lib.bhi_ans_encode_capacity(ns) == wave64.ans_capacity(ns)


# ----------------------------------------------------------------------------- nibble codec in the wave64 layout

@pytest.mark.parametrize("kind,M,K,n", [("gauss", 64, 1024, 1), ("t3", 32, 768, 2), ("bits", 16, 384, 1),
                                        ("special", 32, 512, 1), ("zeros", 8, 384, 1)])
def test_wave64_nibble_round_trip(kind, M, K, n):
    makers = {"gauss": gaussian_weight, "t3": student_t_weight, "bits": random_bits_weight,
              "special": special_values_weight, "zeros": lambda M, K, seed=0: torch.zeros(M, K, dtype=torch.bfloat16)}
    bits = bits_of(makers[kind](M, K, seed=2))
    _, exp = planes.split_bf16(bits)
    base = wave64.nibble_base(np.bincount(exp.reshape(-1), minlength=256))
    enc = wave64.encode_nibble(bits, n, base)
    assert np.array_equal(wave64.decode_nibble(enc["rem"], enc["exp"], enc["offsets"], base), bits)
    inside = ((exp >= base) & (exp < base + 15)).sum()
    words = len(enc["exp"]) - wave64.TAIL_PAD_WORDS
    assert words * 4 >= exp.size // 2 + 4 * (exp.size - inside)          # half a byte each + a word per outlier


def test_nibble_base_is_the_first_best_window():
    c = np.zeros(256, dtype=np.int64)
    c[100:120] = np.arange(20)
    assert wave64.nibble_base(c) == max(range(242), key=lambda b: (c[b:b + 15].sum(), -b)) == 105
    c[:] = 1
    assert wave64.nibble_base(c) == 0
    from bf16_huffman_infer_amd.functional import NibbleCodec
    for seed in range(3):
        h = np.random.default_rng(seed).integers(0, 1000, 256)
        assert NibbleCodec(torch.from_numpy(h)).base == wave64.nibble_base(h)


def test_nibble_capacity_matches_library():
    from bf16_huffman_infer_amd import _lib
    lib = _lib.load()
    for ns in (1, 4, 28, 37, 128):
        assert lib.bhi_nibble_encode_capacity(ns) == wave64.nibble_capacity(ns)

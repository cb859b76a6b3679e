"""The reference's own compressed layout and decoders in numpy (oracle; test
infrastructure only).  This is also the "reference CPU path" timed by ``bench.py``:
the reference itself has no CPU tensor path (every entry asserts ``cuda``,
``functional.py:48,103``), so its decoder is restated here.

Layout (``functional.py:129-242,297-310``):

* row ``(k, r)`` of a split has 64 exponent streams; stream ``g`` carries the symbols of
  columns ``k*Ks + c*128 + 2g + e`` ordered by chunk ``c`` then ``e`` (``:171``);
* each stream is entropy coded on its own, LSB first, into little-endian 32-bit words;
  a row takes ``Wr = max_g words(g)`` words per stream and word ``w`` of stream ``g`` sits
  at ``exp[offsets[k, r] + 64*w + g]`` (``:144-147,175-176``);
* rows are concatenated split-major, in parts of 4096 rows, every part followed by 64
  zero words (``:177,202-231``); ``offsets`` is the running word count;
* inside each 128-column chunk of ``rem``, column ``h*64 + 2l + e`` is stored at byte
  ``4l + 2h + e`` (``:184``).

Decoders (``src/kernel.cu``): Huffman ``:354-380`` (refill 32 bits when fewer than 32 are
valid, four-level byte-table cascade, shift by the code length); rANS ``:652-683`` (state
= first word; refill ``state = state<<32 | word`` when ``state < 256``; ``slot = state &
255``; ``state = freq*(state>>8) + rem``); encoders ``:590-610`` and ``:767-811``;
reassembly ``:293-306`` (lane l: columns 2l,2l+1 from stream l and 64+2l,64+2l+1 from
stream l+32 -- which the per-stream column rule above already implies).

Pins: ``decode(encode(x)) == x`` on seeded Gaussian, Student-t and special-value
tensors; the stream/rem permutations against the index facts recorded for the layout
(stream 0 of Ks=256 = columns [0,1,128,129], stream 33 = [66,67,194,195]; rem byte 0..3
of a chunk = columns [0,1,64,65]); the single-symbol rANS example (stream [1] with the
``ans.py:152`` tables encodes to the word 576); agreement with the wave64 model (both
must give back the same tensor).
"""
import numpy as np

from .planes import rebuild_bf16, split_bf16

STREAMS = 64
PART_ROWS = 4096


def stream_order(exp: np.ndarray) -> np.ndarray:
    """[R, Ks] -> [R, 64, Ks/64]: the symbols of each of the 64 streams of every row."""
    R, Ks = exp.shape
    return exp.reshape(R, Ks // 128, STREAMS, 2).transpose(0, 2, 1, 3).reshape(R, STREAMS, Ks // 64)


def stream_order_inverse(sym: np.ndarray) -> np.ndarray:
    R, _, L = sym.shape
    return sym.reshape(R, STREAMS, L // 2, 2).transpose(0, 2, 1, 3).reshape(R, L * STREAMS)


def permute_rem(rem: np.ndarray) -> np.ndarray:
    R, Ks = rem.shape
    return rem.reshape(R, Ks // 128, 2, 32, 2).transpose(0, 1, 3, 2, 4).reshape(R, Ks)


def permute_rem_inverse(rem: np.ndarray) -> np.ndarray:
    R, Ks = rem.shape
    return rem.reshape(R, Ks // 128, 32, 2, 2).transpose(0, 1, 3, 2, 4).reshape(R, Ks)


# ----------------------------------------------------------------------------- encoders

def _huffman_words(sym: np.ndarray, codes):
    """sym [S, L] -> (words [S, Wmax] uint32, words used per stream)."""
    code_of = np.zeros(256, dtype=np.uint64)
    len_of = np.zeros(256, dtype=np.int64)
    for s, (code, ln) in codes.items():
        code_of[s], len_of[s] = code, ln
    ln = len_of[sym]
    end = np.cumsum(ln, axis=1)
    off = end - ln
    nwords = (end[:, -1] + 31) // 32
    words = np.zeros((sym.shape[0], int(nwords.max()) + 2), dtype=np.uint64)
    rows = np.broadcast_to(np.arange(sym.shape[0])[:, None], sym.shape)
    val = code_of[sym] << (off & 31).astype(np.uint64)          # code <= 32 bits, shift <= 31
    np.bitwise_or.at(words, (rows, off >> 5), val & np.uint64(0xFFFFFFFF))
    np.bitwise_or.at(words, (rows, (off >> 5) + 1), val >> np.uint64(32))
    return words.astype(np.uint32), nwords


def _ans_words(sym: np.ndarray, freq: np.ndarray, cum: np.ndarray):
    """Reverse-order rANS per stream, words reversed into decode order."""
    S, L = sym.shape
    U = np.uint64
    state = np.full(S, 256, dtype=np.uint64)
    rev = np.zeros((S, L + 2), dtype=np.uint32)                  # words in emission order
    n = np.zeros(S, dtype=np.int64)
    rows = np.arange(S)
    f_of = freq.astype(np.uint64)
    c_of = cum.astype(np.uint64)
    for i in range(L - 1, -1, -1):
        f, c = f_of[sym[:, i]], c_of[sym[:, i]]
        emit = (state >> U(32)) >= f                             # state < 2**40: one word at most
        rev[rows[emit], n[emit]] = (state[emit] & U(0xFFFFFFFF)).astype(np.uint32)
        n += emit
        state = np.where(emit, state >> U(32), state)
        state = ((state // f) << U(8)) + (state % f) + c
    for _ in range(2):                                           # flush while state > 0
        emit = state > 0
        rev[rows[emit], n[emit]] = (state[emit] & U(0xFFFFFFFF)).astype(np.uint32)
        n += emit
        state = np.where(emit, state >> U(32), state)
    assert (state == 0).all()
    words = np.zeros((S, int(n.max())), dtype=np.uint32)
    col = np.arange(words.shape[1])[None, :]
    src = n[:, None] - 1 - col
    keep = src >= 0
    words[keep] = rev[np.broadcast_to(rows[:, None], src.shape)[keep], src[keep]]
    return words, n


def encode(bits: np.ndarray, split_k: int, algo: str, tables):
    """bits uint16 [M, K] -> dict(rem [split_k, M, Ks], exp int32, offsets [split_k, M]).

    ``tables``: Huffman ``codes`` dict, or rANS ``(freq, cum)``.
    """
    M, K = bits.shape
    Ks = K // split_k
    rem, exp = split_bf16(bits)
    rem_out = np.zeros((split_k, M, Ks), dtype=np.uint8)
    offsets = np.zeros((split_k, M), dtype=np.int64)
    parts, cursor = [], 0
    for k in range(split_k):
        cols = slice(k * Ks, (k + 1) * Ks)
        rem_out[k] = permute_rem(rem[:, cols])
        for r0 in range(0, M, PART_ROWS):
            sym = stream_order(exp[r0:r0 + PART_ROWS, cols])
            R, _, L = sym.shape
            flat = sym.reshape(R * STREAMS, L)
            words, used = (_huffman_words(flat, tables) if algo == "huffman"
                           else _ans_words(flat, tables[0], tables[1]))
            row_words = used.reshape(R, STREAMS).max(axis=1)
            words = words.reshape(R, STREAMS, -1)
            for r in range(R):
                offsets[k, r0 + r] = cursor
                parts.append(np.ascontiguousarray(words[r, :, :row_words[r]].T).reshape(-1))
                cursor += STREAMS * int(row_words[r])
            parts.append(np.zeros(STREAMS, dtype=np.uint32))
            cursor += STREAMS
    return {"rem": rem_out, "exp": np.concatenate(parts).view(np.int32), "offsets": offsets.astype(np.int32)}


# ----------------------------------------------------------------------------- decoders

def decode_huffman(rem: np.ndarray, exp_words: np.ndarray, offsets: np.ndarray,
                   luts: np.ndarray, lens: np.ndarray) -> np.ndarray:
    """All ``split_k*M*64`` streams in lock step, one symbol per iteration."""
    split_k, M, Ks = rem.shape
    words = exp_words.view(np.uint32).astype(np.uint64)
    U = np.uint64
    ptr = (offsets.astype(np.int64).reshape(-1, 1) + np.arange(STREAMS)).reshape(-1)
    state = np.zeros(ptr.shape, dtype=np.uint64)
    valid = np.zeros(ptr.shape, dtype=np.int64)
    L = Ks // 64
    sym = np.zeros((ptr.shape[0], L), dtype=np.uint8)
    lens64 = lens.astype(np.int64)
    limit = len(words) - 1
    for i in range(L):
        need = valid < 32
        state = np.where(need, state | (words[np.minimum(ptr, limit)] << valid.astype(np.uint64)), state)
        ptr = np.where(need, ptr + STREAMS, ptr)
        valid = np.where(need, valid + 32, valid)
        s = luts[0][(state & U(0xFF)).astype(np.int64)]
        for level in (1, 2, 3):
            miss = s == 255
            if not miss.any():
                break
            nxt = luts[level][((state >> U(8 * level)) & U(0xFF)).astype(np.int64)]
            s = np.where(miss, nxt, s)
        ln = lens64[s]
        state = state >> ln.astype(np.uint64)
        valid = valid - ln
        sym[:, i] = s
    exp = stream_order_inverse(sym.reshape(split_k * M, STREAMS, L)).reshape(split_k, M, Ks)
    return _assemble(rem, exp)


def decode_ans(rem: np.ndarray, exp_words: np.ndarray, offsets: np.ndarray, lut: np.ndarray) -> np.ndarray:
    split_k, M, Ks = rem.shape
    words = exp_words.view(np.uint32).astype(np.uint64)
    U = np.uint64
    ptr = (offsets.astype(np.int64).reshape(-1, 1) + np.arange(STREAMS)).reshape(-1)
    state = words[ptr]
    ptr = ptr + STREAMS
    L = Ks // 64
    sym = np.zeros((ptr.shape[0], L), dtype=np.uint8)
    lut64 = lut.view(np.uint32).astype(np.uint64)
    limit = len(words) - 1
    for i in range(L):
        need = state < U(256)
        state = np.where(need, (state << U(32)) | words[np.minimum(ptr, limit)], state)
        ptr = np.where(need, ptr + STREAMS, ptr)
        e = lut64[(state & U(255)).astype(np.int64)]
        state = ((e >> U(12)) & U(0xFFF)) * (state >> U(8)) + (e & U(0xFFF))
        sym[:, i] = (e >> U(24)).astype(np.uint8)
    exp = stream_order_inverse(sym.reshape(split_k * M, STREAMS, L)).reshape(split_k, M, Ks)
    return _assemble(rem, exp)


def _assemble(rem: np.ndarray, exp: np.ndarray) -> np.ndarray:
    split_k, M, Ks = rem.shape
    out = np.zeros((M, split_k * Ks), dtype=np.uint16)
    for k in range(split_k):
        out[:, k * Ks:(k + 1) * Ks] = rebuild_bf16(permute_rem_inverse(rem[k]), exp[k])
    return out

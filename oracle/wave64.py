"""Executable specification of the wave64 compressed-exponent format (oracle; test
infrastructure only -- the product never imports this file).

The reference stores 64 private bitstreams per row, padded to the longest one
(``functional.py:129-193``), and decodes them with one 32-lane warp per row
(``src/kernel.cu:222-310,354-380``).  The HIP kernels of this repository use a
different private layout with the same planes and the same module buffers:

planes      ``exp`` = BF16 bits 14..7, ``rem`` = sign<<7 | mantissa (reference
            ``utils.py:7-12``); ``split_k`` contiguous column blocks of ``Ks`` columns
            (reference ``functional.py:200``).
row group   4 consecutive rows.  One wavefront decodes one *task* = (split k, row
            group g, chunk c): rows 4g..4g+3, columns ``k*Ks + 128*t + ...`` for the
            steps ``t`` of the chunk.
step        128 columns x 4 rows.  Lane ``l = 4*b + i`` owns row ``4g+i`` and the 8
            columns ``128*t + 8*b + j`` (j = 0..7): 4 exponent *pairs* per step.
rem plane   uint8 ``[split_k, M, Ks]``; the ``4*Ks`` bytes of (k, g) hold step ``t``,
            lane ``l``, column ``j`` at byte ``512*t + 8*l + j``.
code        one length-limited (<= 11 bit) Huffman code over exponent *pairs*
            ``a | b<<8`` (a = even column) plus an ESC word; code bits are consumed
            LSB first.  ``dec`` is the 2048-entry decode table indexed by the next 11
            stream bits: ``len | a<<7 | b<<23`` (the exponents sit where a packed BF16
            pair needs them); ESC entries are ``len | 1<<31``.  The two raw exponents
            of an escaped pair are not in the bitstream: they sit in the task's
            escape list.
lane bits   a lane's codes are concatenated from bit 2 of its private bitstring (the
            decoder keeps its window shifted left by two so that ``window & 0x1FFC`` is
            the byte address of the table entry) and the bitstring is cut into
            32-bit words.
task block  ``[W rows of 64 words][escape list][zero pad]``, a multiple of 4 words:
            word ``w`` of lane ``l`` sits at ``64*w + l`` and ``W`` is the longest lane of
            the task (shorter lanes are zero padded).  Lanes at different depths
            read different rows, but row ``w`` of lane ``l`` always falls into LDS bank
            ``l mod 32``: the per-step window reads are conflict free.  Escape entries
            ``a | b<<8`` are consumed per step in (pair, lane) order and stored
            backwards from the end of the task block.
offsets     int32 ``[split_k, M]``: word offset of task (k, g, c) at ``[k, 4*g + c]``;
            tasks are laid out in (k, g, c) order; unused slots are 0.

Pins: ``decode(encode(x)) == x`` on random, heavy-tailed, constant, all-escape and
boundary inputs, with the encoder (closed-form positions by prefix sums) and the
decoder (step-by-step simulation of the kernel) sharing no code beyond the
constants; cross-check against ``ref_layout`` (both must reproduce the same
original tensor); the HIP encoder must reproduce ``encode`` bit for bit and the
HIP decoder must reproduce the original tensor.
"""
import numpy as np

LANES = 64
GROUP_ROWS = 4
LANE_COLS = 8
STEP_COLS = 128
PAIRS_PER_STEP = 4
WINDOW_WORDS = 3           # words of its bitstring a lane looks at per step
HEADER_BITS = 2            # dummy bits in front of every lane's codes
TABLE_BITS = 11
ESC_FLAG = 1 << 31
TARGET_TASKS = 6144        # wavefronts one MI355X keeps resident: 256 CUs x 4 SIMDs x 6
MIN_CHUNK_STEPS = 4
MAX_CHUNKS = 4
ALIGN_WORDS = 4
TAIL_PAD_WORDS = 2048
ESC_INDEX = 65536          # slot of the ESC code in the encoder table


def chunks_per_group(M: int, Ks: int, split_k: int) -> int:
    """How many independent streams a (split, row group) is cut into."""
    steps = Ks // STEP_COLS
    nc = 1
    while (nc < MAX_CHUNKS and (M // GROUP_ROWS) * split_k * nc * 2 <= TARGET_TASKS
           and steps // (nc * 2) >= MIN_CHUNK_STEPS):
        nc *= 2
    # a row group's tasks are dealt to four wavefronts: a count above four that is no multiple of
    # four would leave them with unequal shares, so it is doubled once more
    if split_k * nc > 4 and (split_k * nc) % 4 != 0 and nc < MAX_CHUNKS and steps // (nc * 2) >= MIN_CHUNK_STEPS:
        nc *= 2
    return nc


def chunk_steps(steps: int, nc: int, c: int):
    return (steps * c) // nc, (steps * (c + 1)) // nc


def lane_order(plane: np.ndarray, split_k: int) -> np.ndarray:
    """[M, K] byte plane -> [split_k, G, S, 64, 8] in (split, group, step, lane, col)."""
    M, K = plane.shape
    Ks = K // split_k
    assert M % GROUP_ROWS == 0 and Ks % STEP_COLS == 0
    G, S = M // GROUP_ROWS, Ks // STEP_COLS
    x = plane.reshape(G, GROUP_ROWS, split_k, S, 16, LANE_COLS)      # g i k t b j
    return np.ascontiguousarray(x.transpose(2, 0, 3, 4, 1, 5)).reshape(split_k, G, S, LANES, LANE_COLS)


def lane_order_inverse(x: np.ndarray) -> np.ndarray:
    split_k, G, S = x.shape[:3]
    y = x.reshape(split_k, G, S, 16, GROUP_ROWS, LANE_COLS).transpose(1, 4, 0, 2, 3, 5)  # g i k t b j
    return np.ascontiguousarray(y).reshape(G * GROUP_ROWS, split_k * S * STEP_COLS)


def pack_rem(rem: np.ndarray, split_k: int) -> np.ndarray:
    M, K = rem.shape
    return lane_order(rem, split_k).reshape(split_k, M, K // split_k)


def unpack_rem(rem_packed: np.ndarray) -> np.ndarray:
    split_k, M, Ks = rem_packed.shape
    return lane_order_inverse(rem_packed.reshape(split_k, M // GROUP_ROWS, Ks // STEP_COLS, LANES, LANE_COLS))


# ----------------------------------------------------------------------------- encoder

def _encode_tasks(sym: np.ndarray, enc: np.ndarray):
    """sym: uint8 [nt, ns, 64, 8] -> list of nt uint32 streams."""
    nt, ns = sym.shape[:2]
    s = sym.astype(np.uint32)
    pairs = s[..., 0::2] | (s[..., 1::2] << 8)                      # [nt, ns, 64, 4]
    e = enc[pairs].astype(np.uint64)
    ln = (e >> np.uint64(16)).astype(np.int64)
    esc = ln == 0                                                    # [nt, ns, 64, 4]
    esc_code = np.uint64(int(enc[ESC_INDEX]) & 0xFFFF)
    esc_len = int(enc[ESC_INDEX]) >> 16
    assert 1 <= esc_len <= TABLE_BITS
    code = np.where(esc, esc_code, e & np.uint64(0xFFFF))
    ln = np.where(esc, esc_len, ln)
    assert ln.max() <= TABLE_BITS and ln.min() >= 1

    # per-lane bit strings
    ln_l = ln.transpose(0, 2, 1, 3).reshape(nt, LANES, ns * PAIRS_PER_STEP)
    code_l = code.transpose(0, 2, 1, 3).reshape(nt, LANES, ns * PAIRS_PER_STEP)
    end = HEADER_BITS + np.cumsum(ln_l, axis=-1)
    off = end - ln_l
    nwords = (end[..., -1] + 31) // 32                               # [nt, 64]
    rows = nwords.max(axis=-1)                                       # [nt]
    lw = np.zeros((nt, LANES, int(rows.max()) + 1), dtype=np.uint64)
    ti, li, _ = np.indices(off.shape)
    val = code_l << (off & 31).astype(np.uint64)
    np.bitwise_or.at(lw, (ti, li, off >> 5), val & np.uint64(0xFFFFFFFF))
    np.bitwise_or.at(lw, (ti, li, (off >> 5) + 1), val >> np.uint64(32))

    esc_flat = esc.transpose(0, 1, 3, 2).reshape(nt, -1)             # (step, pair, lane) order
    pair_flat = pairs.transpose(0, 1, 3, 2).reshape(nt, -1)
    nesc = esc_flat.sum(axis=-1)

    streams = []
    for t in range(nt):
        body = int(rows[t]) * LANES + int(nesc[t])
        total = (body + ALIGN_WORDS - 1) // ALIGN_WORDS * ALIGN_WORDS
        st = np.zeros(total, dtype=np.uint32)
        st[:int(rows[t]) * LANES] = lw[t, :, :int(rows[t])].T.reshape(-1).astype(np.uint32)
        if nesc[t]:
            st[total - 1 - np.arange(int(nesc[t]))] = pair_flat[t][esc_flat[t]]
        streams.append(st)
    return streams


def encode(bits: np.ndarray, split_k: int, enc: np.ndarray):
    """bits: uint16 [M, K] BF16 patterns -> dict(rem, exp, offsets, nc)."""
    from .planes import split_bf16
    M, K = bits.shape
    Ks = K // split_k
    S = Ks // STEP_COLS
    G = M // GROUP_ROWS
    nc = chunks_per_group(M, Ks, split_k)
    rem, exp = split_bf16(bits)
    sym = lane_order(exp, split_k)                                   # [k, G, S, 64, 8]
    per_chunk = []
    for c in range(nc):
        t0, t1 = chunk_steps(S, nc, c)
        per_chunk.append(_encode_tasks(sym[:, :, t0:t1].reshape(split_k * G, t1 - t0, LANES, LANE_COLS), enc))
    offsets = np.zeros((split_k, M), dtype=np.int64)
    parts, cursor = [], 0
    for k in range(split_k):
        for g in range(G):
            for c in range(nc):
                st = per_chunk[c][k * G + g]
                offsets[k, GROUP_ROWS * g + c] = cursor
                parts.append(st)
                cursor += len(st)
    parts.append(np.zeros(TAIL_PAD_WORDS, dtype=np.uint32))
    assert cursor + TAIL_PAD_WORDS < 2 ** 31
    return {
        "rem": pack_rem(rem, split_k),
        "exp": np.concatenate(parts).view(np.int32),
        "offsets": offsets.astype(np.int32),
        "nc": nc,
    }


# ----------------------------------------------------------------------------- decoder

def _decode_tasks(words: np.ndarray, base: np.ndarray, end: np.ndarray, ns: int, dec: np.ndarray) -> np.ndarray:
    """Step-by-step model of one wavefront per task.

    words: uint32 flat buffer; base/end: [nt] word offsets of each task block and of
    the block that follows it.  Returns uint8 [nt, ns, 64, 8].
    """
    nt = len(base)
    U = np.uint64
    lanes = np.arange(LANES)
    w64 = words.astype(np.uint64)
    pos = np.zeros((nt, LANES), dtype=np.int64)        # cursor = bit position - 2 (the window is pre-shifted)
    eptr = np.zeros(nt, dtype=np.int64)
    out = np.zeros((nt, ns, LANES, LANE_COLS), dtype=np.uint8)
    dec64 = dec.astype(np.uint64)
    M32 = U(0xFFFFFFFF)
    for t in range(ns):
        row = pos >> 5
        at = base[:, None] + row * LANES + lanes
        lo, hi, nx = w64[at], w64[at + LANES], w64[at + 2 * LANES]
        cu = (pos & 31).astype(np.uint64)
        wlo = (((hi << U(32)) | lo) >> cu) & M32
        whi = (((nx << U(32)) | hi) >> cu) & M32
        win = (whi << U(32)) | wlo
        for q in range(PAIRS_PER_STEP):
            e = dec64[((win >> U(HEADER_BITS)) & U((1 << TABLE_BITS) - 1)).astype(np.int64)]
            ln = (e & U(0x1F)).astype(np.int64)
            esc = ((e >> U(31)) & U(1)).astype(bool)
            a = ((e >> U(7)) & U(0xFF)).astype(np.uint8)
            b = ((e >> U(23)) & U(0xFF)).astype(np.uint8)
            if esc.any():
                rank = np.cumsum(esc, axis=-1) - esc
                src = end[:, None] - 1 - (eptr[:, None] + rank)
                v = words[np.where(esc, src, 0)]
                a = np.where(esc, (v & 0xFF).astype(np.uint8), a)
                b = np.where(esc, ((v >> 8) & 0xFF).astype(np.uint8), b)
                eptr += esc.sum(axis=-1)
            out[:, t, :, 2 * q] = a
            out[:, t, :, 2 * q + 1] = b
            win = win >> ln.astype(np.uint64)
            pos = pos + ln
    return out


def decode(rem_packed: np.ndarray, exp_words: np.ndarray, offsets: np.ndarray, dec: np.ndarray) -> np.ndarray:
    """-> uint16 [M, K] BF16 patterns."""
    from .planes import rebuild_bf16
    split_k, M, Ks = rem_packed.shape
    S, G = Ks // STEP_COLS, M // GROUP_ROWS
    nc = chunks_per_group(M, Ks, split_k)
    words = exp_words.view(np.uint32)
    total = len(words) - TAIL_PAD_WORDS
    off = offsets.astype(np.int64).reshape(split_k, G, GROUP_ROWS)[:, :, :nc]   # [k, G, nc] in layout order
    flat = off.reshape(-1)
    nxt = np.concatenate([flat[1:], [total]]).reshape(off.shape)
    sym = np.zeros((split_k, G, S, LANES, LANE_COLS), dtype=np.uint8)
    for c in range(nc):
        t0, t1 = chunk_steps(S, nc, c)
        r = _decode_tasks(words, off[:, :, c].reshape(-1), nxt[:, :, c].reshape(-1), t1 - t0, dec)
        sym[:, :, t0:t1] = r.reshape(split_k, G, t1 - t0, LANES, LANE_COLS)
    exp = lane_order_inverse(sym)
    rem = unpack_rem(rem_packed)
    return rebuild_bf16(rem, exp)


# ----------------------------------------------------------------------------- rANS codec
#
# Same planes, tasks, lanes, rows and offsets as the Huffman stream; a task block is
# ``[W rows of 64 words][zero pad]`` with no escape list.  Each lane owns ONE rANS state
# (64 bit, precision 8, 32-bit renormalisation words), i.e. the reference's state and
# tables (``src/kernel.cu:652-683``, ``ans.py:6-80``) with a different renormalisation
# schedule: the decoder looks at its state only after every FOUR symbols (the two halves
# of a step) and pulls one word when the state has dropped below 2**32.  Decoding is the
# exact inverse of encoding for any state value, so four symbols may be taken without a
# refill; the encoder (which runs backwards) emits the low word of its state before a
# half-step whenever encoding the four symbols would overflow 64 bits or the decoder
# would see a state below 2**32.  Rows 0 and 1 of a lane are its initial state.

ANS_PRECISION = 8
ANS_HALF = 4                   # symbols between two refill checks
ANS_INIT_ROWS = 2


def ans_capacity(n_steps: int) -> int:
    return LANES * (2 * n_steps + ANS_INIT_ROWS) + ALIGN_WORDS


def _ans_encode_tasks(sym: np.ndarray, freq: np.ndarray, cum: np.ndarray):
    """sym: uint8 [nt, ns, 64, 8] -> list of nt uint32 task blocks."""
    nt, ns = sym.shape[:2]
    U = np.uint64
    f_of, c_of = freq.astype(np.uint64), cum.astype(np.uint64)
    assert (f_of[np.unique(sym)] > 0).all(), "symbol without a frequency"
    x = np.full((nt, LANES), 1 << 32, dtype=np.uint64)
    rev = np.zeros((nt, LANES, 2 * ns + ANS_INIT_ROWS), dtype=np.uint32)        # emission order
    n = np.zeros((nt, LANES), dtype=np.int64)
    ti, li = np.indices((nt, LANES))

    def emit(mask, value):
        rev[ti[mask], li[mask], n[mask]] = value[mask].astype(np.uint32)
        n[mask] += 1

    for t in range(ns - 1, -1, -1):
        for half in (1, 0):
            s4 = sym[:, t, :, ANS_HALF * half:ANS_HALF * (half + 1)].astype(np.int64)    # [nt, 64, 4]
            # would the four symbols fit without a refill?
            y, fits = x.copy(), x >= U(1 << 32)
            for j in range(ANS_HALF - 1, -1, -1):
                f, c = f_of[s4[..., j]], c_of[s4[..., j]]
                q = y // f
                fits &= q < U(1 << 56)
                y = ((q & U((1 << 56) - 1)) << U(8)) + (y % f) + c
            must = ~fits
            emit(must, x & U(0xFFFFFFFF))
            x = np.where(must, x >> U(32), x)
            for j in range(ANS_HALF - 1, -1, -1):
                f, c = f_of[s4[..., j]], c_of[s4[..., j]]
                x = ((x // f) << U(8)) + (x % f) + c
    every = np.ones((nt, LANES), dtype=bool)
    emit(every, x >> U(32))
    emit(every, x & U(0xFFFFFFFF))

    rows = n.max(axis=-1)
    blocks = []
    for t in range(nt):
        W = int(rows[t])
        total = (W * LANES + ALIGN_WORDS - 1) // ALIGN_WORDS * ALIGN_WORDS
        blk = np.zeros(total, dtype=np.uint32)
        lw = np.zeros((LANES, W), dtype=np.uint32)
        col = np.arange(W)[None, :]
        src = n[t][:, None] - 1 - col                               # decode order = reverse emission
        keep = src >= 0
        lw[keep] = rev[t][np.broadcast_to(np.arange(LANES)[:, None], src.shape)[keep], src[keep]]
        blk[:W * LANES] = lw.T.reshape(-1)
        blocks.append(blk)
    return blocks


def _ans_decode_tasks(words: np.ndarray, base: np.ndarray, ns: int, lut: np.ndarray) -> np.ndarray:
    """Step-by-step model of one wavefront per task.  lut: uint32[256] packed
    (sym<<24)|(freq<<12)|rem."""
    nt = len(base)
    U = np.uint64
    lanes = np.arange(LANES)
    w64 = words.astype(np.uint64)
    lut64 = lut.astype(np.uint64)
    at = base[:, None] + lanes
    x = w64[at] | (w64[at + LANES] << U(32))
    row = np.full((nt, LANES), ANS_INIT_ROWS, dtype=np.int64)
    out = np.zeros((nt, ns, LANES, LANE_COLS), dtype=np.uint8)
    limit = len(words) - 1
    for t in range(ns):
        for half in (0, 1):
            for j in range(ANS_HALF):
                e = lut64[(x & U(0xFF)).astype(np.int64)]
                out[:, t, :, ANS_HALF * half + j] = (e >> U(24)).astype(np.uint8)
                x = ((e >> U(12)) & U(0xFFF)) * (x >> U(8)) + (e & U(0xFFF))
            need = x < U(1 << 32)
            w = w64[np.minimum(base[:, None] + row * LANES + lanes, limit)]
            x = np.where(need, (x << U(32)) | w, x)
            row = row + need
    return out


def encode_ans(bits: np.ndarray, split_k: int, freq: np.ndarray, cum: np.ndarray):
    """bits: uint16 [M, K] BF16 patterns -> dict(rem, exp, offsets, nc)."""
    from .planes import split_bf16
    M, K = bits.shape
    Ks = K // split_k
    S, G = Ks // STEP_COLS, M // GROUP_ROWS
    nc = chunks_per_group(M, Ks, split_k)
    rem, exp = split_bf16(bits)
    sym = lane_order(exp, split_k)
    per_chunk = []
    for c in range(nc):
        t0, t1 = chunk_steps(S, nc, c)
        per_chunk.append(_ans_encode_tasks(sym[:, :, t0:t1].reshape(split_k * G, t1 - t0, LANES, LANE_COLS), freq, cum))
    offsets = np.zeros((split_k, M), dtype=np.int64)
    parts, cursor = [], 0
    for k in range(split_k):
        for g in range(G):
            for c in range(nc):
                blk = per_chunk[c][k * G + g]
                offsets[k, GROUP_ROWS * g + c] = cursor
                parts.append(blk)
                cursor += len(blk)
    parts.append(np.zeros(TAIL_PAD_WORDS, dtype=np.uint32))
    return {"rem": pack_rem(rem, split_k), "exp": np.concatenate(parts).view(np.int32),
            "offsets": offsets.astype(np.int32), "nc": nc}


def decode_ans(rem_packed: np.ndarray, exp_words: np.ndarray, offsets: np.ndarray, lut: np.ndarray) -> np.ndarray:
    """-> uint16 [M, K] BF16 patterns."""
    from .planes import rebuild_bf16
    split_k, M, Ks = rem_packed.shape
    S, G = Ks // STEP_COLS, M // GROUP_ROWS
    nc = chunks_per_group(M, Ks, split_k)
    words = exp_words.view(np.uint32)
    off = offsets.astype(np.int64).reshape(split_k, G, GROUP_ROWS)[:, :, :nc]
    sym = np.zeros((split_k, G, S, LANES, LANE_COLS), dtype=np.uint8)
    for c in range(nc):
        t0, t1 = chunk_steps(S, nc, c)
        r = _ans_decode_tasks(words, off[:, :, c].reshape(-1), t1 - t0, lut.view(np.uint32))
        sym[:, :, t0:t1] = r.reshape(split_k, G, t1 - t0, LANES, LANE_COLS)
    return rebuild_bf16(unpack_rem(rem_packed), lane_order_inverse(sym))


# ----------------------------------------------------------------------------- nibble codec
#
# A fixed-width code (not in the reference): every exponent inside a window of 15
# consecutive values ``[base, base + 14]`` is stored as the 4-bit offset from ``base``,
# anything else as the nibble 15 plus one word of the task's escape list.  Same planes,
# tasks, lanes and offsets as the other codecs; a task block is
# ``[ns rows of 64 words][escape list][zero pad]``: row ``t``, lane ``l`` holds the eight
# nibbles of the lane's columns of step ``t`` (column ``j`` in bits ``4j..4j+3``).  Escape
# words (the raw exponent) are consumed per step in (column, lane) order and stored
# backwards from the end of the block.  Nothing is variable-length inside a block, so
# the decoder needs no table, no cursor and no serial dependency.

NIBBLE_ESC = 15


def nibble_base(counts: np.ndarray) -> int:
    """Start of the 15-wide exponent window that covers the most weights (first best)."""
    c = np.asarray(counts, dtype=np.int64)
    cover = np.convolve(c, np.ones(NIBBLE_ESC, dtype=np.int64))[NIBBLE_ESC - 1:NIBBLE_ESC - 1 + 256 - NIBBLE_ESC + 1]
    return int(np.argmax(cover))


def nibble_capacity(n_steps: int) -> int:
    return n_steps * LANES + n_steps * LANE_COLS * LANES + ALIGN_WORDS


def _nibble_encode_tasks(sym: np.ndarray, base: int):
    """sym: uint8 [nt, ns, 64, 8] -> list of nt uint32 task blocks."""
    nt, ns = sym.shape[:2]
    off = sym.astype(np.int64) - base
    esc = (off < 0) | (off >= NIBBLE_ESC)
    nib = np.where(esc, NIBBLE_ESC, off).astype(np.uint32)
    rows = np.zeros((nt, ns, LANES), dtype=np.uint32)
    for j in range(LANE_COLS):
        rows |= nib[..., j] << np.uint32(4 * j)
    esc_flat = esc.transpose(0, 1, 3, 2).reshape(nt, -1)             # (step, column, lane) order
    raw_flat = sym.transpose(0, 1, 3, 2).reshape(nt, -1).astype(np.uint32)
    blocks = []
    for t in range(nt):
        nesc = int(esc_flat[t].sum())
        total = (ns * LANES + nesc + ALIGN_WORDS - 1) // ALIGN_WORDS * ALIGN_WORDS
        blk = np.zeros(total, dtype=np.uint32)
        blk[:ns * LANES] = rows[t].reshape(-1)
        if nesc:
            blk[total - 1 - np.arange(nesc)] = raw_flat[t][esc_flat[t]]
        blocks.append(blk)
    return blocks


def _nibble_decode_tasks(words: np.ndarray, base_w: np.ndarray, end_w: np.ndarray, ns: int, base: int) -> np.ndarray:
    nt = len(base_w)
    lanes = np.arange(LANES)
    out = np.zeros((nt, ns, LANES, LANE_COLS), dtype=np.uint8)
    eptr = np.zeros(nt, dtype=np.int64)
    for t in range(ns):
        d = words[base_w[:, None] + t * LANES + lanes]
        for j in range(LANE_COLS):
            n = (d >> np.uint32(4 * j)) & np.uint32(15)
            esc = n == NIBBLE_ESC
            val = (n + np.uint32(base)).astype(np.uint8)
            if esc.any():
                rank = np.cumsum(esc, axis=-1) - esc
                src = end_w[:, None] - 1 - (eptr[:, None] + rank)
                raw = words[np.where(esc, src, 0)]
                val = np.where(esc, raw.astype(np.uint8), val)
                eptr += esc.sum(axis=-1)
            out[:, t, :, j] = val
    return out


def encode_nibble(bits: np.ndarray, split_k: int, base: int):
    """bits: uint16 [M, K] BF16 patterns -> dict(rem, exp, offsets, nc)."""
    from .planes import split_bf16
    M, K = bits.shape
    Ks = K // split_k
    S, G = Ks // STEP_COLS, M // GROUP_ROWS
    nc = chunks_per_group(M, Ks, split_k)
    rem, exp = split_bf16(bits)
    sym = lane_order(exp, split_k)
    per_chunk = []
    for c in range(nc):
        t0, t1 = chunk_steps(S, nc, c)
        per_chunk.append(_nibble_encode_tasks(sym[:, :, t0:t1].reshape(split_k * G, t1 - t0, LANES, LANE_COLS), base))
    offsets = np.zeros((split_k, M), dtype=np.int64)
    parts, cursor = [], 0
    for k in range(split_k):
        for g in range(G):
            for c in range(nc):
                blk = per_chunk[c][k * G + g]
                offsets[k, GROUP_ROWS * g + c] = cursor
                parts.append(blk)
                cursor += len(blk)
    parts.append(np.zeros(TAIL_PAD_WORDS, dtype=np.uint32))
    return {"rem": pack_rem(rem, split_k), "exp": np.concatenate(parts).view(np.int32),
            "offsets": offsets.astype(np.int32), "nc": nc}


def decode_nibble(rem_packed: np.ndarray, exp_words: np.ndarray, offsets: np.ndarray, base: int) -> np.ndarray:
    """-> uint16 [M, K] BF16 patterns."""
    from .planes import rebuild_bf16
    split_k, M, Ks = rem_packed.shape
    S, G = Ks // STEP_COLS, M // GROUP_ROWS
    nc = chunks_per_group(M, Ks, split_k)
    words = exp_words.view(np.uint32)
    total = len(words) - TAIL_PAD_WORDS
    off = offsets.astype(np.int64).reshape(split_k, G, GROUP_ROWS)[:, :, :nc]
    flat = off.reshape(-1)
    nxt = np.concatenate([flat[1:], [total]]).reshape(off.shape)
    sym = np.zeros((split_k, G, S, LANES, LANE_COLS), dtype=np.uint8)
    for c in range(nc):
        t0, t1 = chunk_steps(S, nc, c)
        r = _nibble_decode_tasks(words, off[:, :, c].reshape(-1), nxt[:, :, c].reshape(-1), t1 - t0, base)
        sym[:, :, t0:t1] = r.reshape(split_k, G, t1 - t0, LANES, LANE_COLS)
    return rebuild_bf16(unpack_rem(rem_packed), lane_order_inverse(sym))


# ----------------------------------------------------------------------------- table checks

def check_tables(dec: np.ndarray, enc: np.ndarray) -> None:
    """Consistency of a decode table with its encoder table (raises AssertionError).

    Every table index must resolve to exactly the pair (or ESC) whose LSB-first code
    is a prefix of the index; the code is therefore prefix-free and complete.
    """
    assert dec.shape == (1 << TABLE_BITS,) and enc.shape == (ESC_INDEX + 1,)
    covered = np.zeros(1 << TABLE_BITS, dtype=np.int64)
    present = np.nonzero(enc >> 16)[0]
    kraft = 0.0
    for p in present:
        code, ln = int(enc[p]) & 0xFFFF, int(enc[p]) >> 16
        assert 1 <= ln <= TABLE_BITS and code < (1 << ln)
        kraft += 2.0 ** -ln
        idx = code + (np.arange(1 << (TABLE_BITS - ln)) << ln)
        covered[idx] += 1
        got = dec[idx]
        if p == ESC_INDEX:
            assert (got == (ln | ESC_FLAG)).all()
        else:
            want = ln | ((p & 0xFF) << 7) | ((p >> 8) << 23)
            assert (got == want).all(), (p, ln)
    assert (covered == 1).all()
    assert abs(kraft - 1.0) < 1e-9
    assert enc[ESC_INDEX] >> 16 != 0

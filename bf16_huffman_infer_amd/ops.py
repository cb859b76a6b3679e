"""The six custom ops of namespace ``bf16_huffman_infer`` on HIP (the nibble codec's three live in a
namespace of their own, ``bf16_huffman_infer_amd``: the reference's namespace carries the reference's schemas only).

Same op names, schemas and positional wrappers as the reference
(``bf16_huffman_infer/src/bf16_huffman_infer.cpp:29-35``, ``ops.py:6-61``).  The schemas
are registered from Python and the ``CUDA`` dispatch key (the key ROCm devices use)
forwards raw device pointers and the current torch stream to ``libbhi_hip.so``.
No other key is registered: CPU tensors are rejected by the dispatcher, as the
reference rejects them with asserts.

Every op mutates caller-allocated outputs and returns nothing; nothing here
synchronises or allocates, so the ops can be captured in a HIP graph.
"""
import torch
from torch import Tensor

from . import _lib

_LIB = torch.library.Library("bf16_huffman_infer", "DEF")
_LIB.define("gemv_bf16_huffman(Tensor A_rem, Tensor A_exp, Tensor X, Tensor(a!) Y, Tensor offsets, "
            "Tensor LUT1, Tensor LUT2, Tensor LUT3, Tensor LUT4, Tensor code_lengths) -> ()")
_LIB.define("huffman_encode(Tensor data, Tensor LUT, Tensor(a!) output, Tensor(b!) output_lengths) -> ()")
_LIB.define("huffman_decode(Tensor A_rem, Tensor A_exp, Tensor(a!) Y, Tensor offsets, "
            "Tensor LUT1, Tensor LUT2, Tensor LUT3, Tensor LUT4, Tensor code_lengths) -> ()")
_LIB.define("gemv_bf16_ans(Tensor A_rem, Tensor A_exp, Tensor X, Tensor(a!) Y, Tensor offsets, Tensor LUT) -> ()")
_LIB.define("ans_encode(Tensor data, Tensor freq, Tensor cum, Tensor(a!) output, Tensor(b!) output_lengths) -> ()")
_LIB.define("ans_decode(Tensor A_rem, Tensor A_exp, Tensor(a!) Y, Tensor offsets, Tensor LUT) -> ()")
# not in the reference, hence not in its namespace: the fixed-width codec, with the rANS ops' shapes
_EXTRA = torch.library.Library("bf16_huffman_infer_amd", "DEF")
_EXTRA.define("gemv_bf16_nibble(Tensor A_rem, Tensor A_exp, Tensor X, Tensor(a!) Y, Tensor offsets, Tensor LUT) -> ()")
_EXTRA.define("nibble_encode(Tensor data, Tensor LUT, Tensor(a!) output, Tensor(b!) output_lengths) -> ()")
_EXTRA.define("nibble_decode(Tensor A_rem, Tensor A_exp, Tensor(a!) Y, Tensor offsets, Tensor LUT) -> ()")

LANE_BYTES_PER_STEP = 512          # 64 lanes x 8 exponent bytes


_ready_devices = set()


def _stream(t: Tensor) -> int:
    """The current torch stream of ``t``'s device.  The first op on a device also lets the
    library do its once-per-device lookups: whatever comes first in a process is an eager call
    (a conversion, a warm-up), so none of them is left for a call under stream capture."""
    device = t.device
    if device not in _ready_devices:
        if not torch.cuda.is_current_stream_capturing():
            with torch.cuda.device(device):
                _lib.check(_lib.load().bhi_device_init(), "device_init")
            _ready_devices.add(device)
    return torch.cuda.current_stream(device).cuda_stream


def _req(t: Tensor, dtype, name: str, ref: Tensor = None) -> int:
    if t.dtype != dtype:
        raise RuntimeError(f"{name}: expected {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise RuntimeError(f"{name}: must be contiguous")
    if ref is not None and t.device != ref.device:
        raise RuntimeError(f"{name}: on {t.device}, expected {ref.device}")
    return t.data_ptr()


def _weight_dims(A_rem: Tensor, offsets: Tensor):
    if A_rem.dim() != 3:
        raise RuntimeError(f"A_rem must be [split_k, M, Ks], got {tuple(A_rem.shape)}")
    split_k, M, Ks = A_rem.shape
    if tuple(offsets.shape) != (split_k, M):
        raise RuntimeError(f"offsets must be [{split_k}, {M}], got {tuple(offsets.shape)}")
    return split_k, M, Ks


def _gemv_common(A_rem, A_exp, X, Y, offsets):
    split_k, M, Ks = _weight_dims(A_rem, offsets)
    if X.dim() != 3 or X.shape[1] != split_k or X.shape[2] != Ks:
        raise RuntimeError(f"X must be [batch, {split_k}, {Ks}], got {tuple(X.shape)}")
    batch = X.shape[0]
    if tuple(Y.shape) != (batch, M):
        raise RuntimeError(f"Y must be [{batch}, {M}], got {tuple(Y.shape)}")
    return split_k, M, Ks, batch


def _gemv_bf16_huffman(A_rem, A_exp, X, Y, offsets, LUT1, LUT2, LUT3, LUT4, code_lengths):
    lib = _lib.load()
    split_k, M, Ks, batch = _gemv_common(A_rem, A_exp, X, Y, offsets)
    with torch.cuda.device(A_rem.device):
        rc = lib.bhi_gemv_bf16_huffman(
            _req(A_rem, torch.uint8, "A_rem"), _req(A_exp, torch.int32, "A_exp", A_rem), A_exp.numel(),
            _req(X, torch.bfloat16, "X", A_rem), _req(Y, torch.bfloat16, "Y", A_rem),
            _req(offsets, torch.int32, "offsets", A_rem),
            _req(LUT1, torch.uint8, "LUT1", A_rem), LUT1.numel(),
            _req(LUT2, torch.uint8, "LUT2", A_rem), _req(LUT3, torch.uint8, "LUT3", A_rem),
            _req(LUT4, torch.uint8, "LUT4", A_rem), _req(code_lengths, torch.uint8, "code_lengths", A_rem),
            split_k, M, Ks, batch, _stream(A_rem))
    _lib.check(rc, "gemv_bf16_huffman")


def _huffman_decode(A_rem, A_exp, Y, offsets, LUT1, LUT2, LUT3, LUT4, code_lengths):
    lib = _lib.load()
    split_k, M, Ks = _weight_dims(A_rem, offsets)
    if tuple(Y.shape) != (M, split_k * Ks):
        raise RuntimeError(f"Y must be [{M}, {split_k * Ks}], got {tuple(Y.shape)}")
    with torch.cuda.device(A_rem.device):
        rc = lib.bhi_huffman_decode(
            _req(A_rem, torch.uint8, "A_rem"), _req(A_exp, torch.int32, "A_exp", A_rem), A_exp.numel(),
            _req(Y, torch.bfloat16, "Y", A_rem), _req(offsets, torch.int32, "offsets", A_rem),
            _req(LUT1, torch.uint8, "LUT1", A_rem), LUT1.numel(),
            _req(LUT2, torch.uint8, "LUT2", A_rem), _req(LUT3, torch.uint8, "LUT3", A_rem),
            _req(LUT4, torch.uint8, "LUT4", A_rem), _req(code_lengths, torch.uint8, "code_lengths", A_rem),
            split_k, M, Ks, _stream(A_rem))
    _lib.check(rc, "huffman_decode")


def _encode_dims(data: Tensor, output: Tensor, output_lengths: Tensor):
    if data.dim() != 2 or data.shape[1] % LANE_BYTES_PER_STEP != 0:
        raise RuntimeError(f"data must be [tasks, steps*512], got {tuple(data.shape)}")
    n_tasks, n_steps = data.shape[0], data.shape[1] // LANE_BYTES_PER_STEP
    if output.dim() != 2 or output.shape[0] != n_tasks or tuple(output_lengths.shape) != (n_tasks,):
        raise RuntimeError("output must be [tasks, stride] and output_lengths [tasks]")
    return n_tasks, n_steps


def _huffman_encode(data, LUT, output, output_lengths):
    lib = _lib.load()
    n_tasks, n_steps = _encode_dims(data, output, output_lengths)
    if LUT.numel() != 65537:
        raise RuntimeError("LUT must hold 65537 encoder entries")
    with torch.cuda.device(data.device):
        rc = lib.bhi_huffman_encode(
            _req(data, torch.uint8, "data"), _req(LUT, torch.int32, "LUT", data),
            _req(output, torch.int32, "output", data), _req(output_lengths, torch.int32, "output_lengths", data),
            n_tasks, n_steps, output.shape[1], _stream(data))
    _lib.check(rc, "huffman_encode")


def _gemv_bf16_ans(A_rem, A_exp, X, Y, offsets, LUT):
    lib = _lib.load()
    split_k, M, Ks, batch = _gemv_common(A_rem, A_exp, X, Y, offsets)
    if LUT.numel() != 256:
        raise RuntimeError("LUT must hold 256 rANS slots")
    with torch.cuda.device(A_rem.device):
        rc = lib.bhi_gemv_bf16_ans(
            _req(A_rem, torch.uint8, "A_rem"), _req(A_exp, torch.int32, "A_exp", A_rem), A_exp.numel(),
            _req(X, torch.bfloat16, "X", A_rem), _req(Y, torch.bfloat16, "Y", A_rem),
            _req(offsets, torch.int32, "offsets", A_rem), _req(LUT, torch.int32, "LUT", A_rem),
            split_k, M, Ks, batch, _stream(A_rem))
    _lib.check(rc, "gemv_bf16_ans")


def _ans_decode(A_rem, A_exp, Y, offsets, LUT):
    lib = _lib.load()
    split_k, M, Ks = _weight_dims(A_rem, offsets)
    if tuple(Y.shape) != (M, split_k * Ks):
        raise RuntimeError(f"Y must be [{M}, {split_k * Ks}], got {tuple(Y.shape)}")
    if LUT.numel() != 256:
        raise RuntimeError("LUT must hold 256 rANS slots")
    with torch.cuda.device(A_rem.device):
        rc = lib.bhi_ans_decode(
            _req(A_rem, torch.uint8, "A_rem"), _req(A_exp, torch.int32, "A_exp", A_rem), A_exp.numel(),
            _req(Y, torch.bfloat16, "Y", A_rem), _req(offsets, torch.int32, "offsets", A_rem),
            _req(LUT, torch.int32, "LUT", A_rem), split_k, M, Ks, _stream(A_rem))
    _lib.check(rc, "ans_decode")


def _ans_encode(data, freq, cum, output, output_lengths):
    lib = _lib.load()
    n_tasks, n_steps = _encode_dims(data, output, output_lengths)
    if freq.numel() != 256 or cum.numel() != 256:
        raise RuntimeError("freq and cum must hold 256 entries")
    with torch.cuda.device(data.device):
        rc = lib.bhi_ans_encode(
            _req(data, torch.uint8, "data"), _req(freq, torch.int32, "freq", data), _req(cum, torch.int32, "cum", data),
            _req(output, torch.int32, "output", data), _req(output_lengths, torch.int32, "output_lengths", data),
            n_tasks, n_steps, output.shape[1], _stream(data))
    _lib.check(rc, "ans_encode")


def _gemv_bf16_nibble(A_rem, A_exp, X, Y, offsets, LUT):
    lib = _lib.load()
    split_k, M, Ks, batch = _gemv_common(A_rem, A_exp, X, Y, offsets)
    if LUT.numel() != 256:
        raise RuntimeError("LUT must hold 256 entries")
    with torch.cuda.device(A_rem.device):
        rc = lib.bhi_gemv_bf16_nibble(
            _req(A_rem, torch.uint8, "A_rem"), _req(A_exp, torch.int32, "A_exp", A_rem), A_exp.numel(),
            _req(X, torch.bfloat16, "X", A_rem), _req(Y, torch.bfloat16, "Y", A_rem),
            _req(offsets, torch.int32, "offsets", A_rem), _req(LUT, torch.int32, "LUT", A_rem),
            split_k, M, Ks, batch, _stream(A_rem))
    _lib.check(rc, "gemv_bf16_nibble")


def _nibble_decode(A_rem, A_exp, Y, offsets, LUT):
    lib = _lib.load()
    split_k, M, Ks = _weight_dims(A_rem, offsets)
    if tuple(Y.shape) != (M, split_k * Ks):
        raise RuntimeError(f"Y must be [{M}, {split_k * Ks}], got {tuple(Y.shape)}")
    if LUT.numel() != 256:
        raise RuntimeError("LUT must hold 256 entries")
    with torch.cuda.device(A_rem.device):
        rc = lib.bhi_nibble_decode(
            _req(A_rem, torch.uint8, "A_rem"), _req(A_exp, torch.int32, "A_exp", A_rem), A_exp.numel(),
            _req(Y, torch.bfloat16, "Y", A_rem), _req(offsets, torch.int32, "offsets", A_rem),
            _req(LUT, torch.int32, "LUT", A_rem), split_k, M, Ks, _stream(A_rem))
    _lib.check(rc, "nibble_decode")


def _nibble_encode(data, LUT, output, output_lengths):
    lib = _lib.load()
    n_tasks, n_steps = _encode_dims(data, output, output_lengths)
    if LUT.numel() != 256:
        raise RuntimeError("LUT must hold 256 entries")
    with torch.cuda.device(data.device):
        rc = lib.bhi_nibble_encode(
            _req(data, torch.uint8, "data"), _req(LUT, torch.int32, "LUT", data),
            _req(output, torch.int32, "output", data), _req(output_lengths, torch.int32, "output_lengths", data),
            n_tasks, n_steps, output.shape[1], _stream(data))
    _lib.check(rc, "nibble_encode")


for _name, _fn in (("gemv_bf16_nibble", _gemv_bf16_nibble), ("nibble_encode", _nibble_encode),
                   ("nibble_decode", _nibble_decode)):
    _EXTRA.impl(_name, _fn, "CUDA")

for _name, _fn in (("gemv_bf16_huffman", _gemv_bf16_huffman), ("huffman_encode", _huffman_encode),
                   ("huffman_decode", _huffman_decode), ("gemv_bf16_ans", _gemv_bf16_ans),
                   ("ans_encode", _ans_encode), ("ans_decode", _ans_decode)):
    _LIB.impl(_name, _fn, "CUDA")


def gemv_bf16_huffman(
    A_rem: Tensor, A_exp: Tensor, X: Tensor, Y: Tensor,
    offsets: Tensor,
    LUT1: Tensor, LUT2: Tensor, LUT3: Tensor, LUT4: Tensor,
    code_lengths: Tensor,
) -> None:
    torch.ops.bf16_huffman_infer.gemv_bf16_huffman.default(
        A_rem, A_exp, X, Y, offsets, LUT1, LUT2, LUT3, LUT4, code_lengths)


def huffman_encode(data: Tensor, LUT: Tensor, output: Tensor, output_lengths: Tensor) -> None:
    torch.ops.bf16_huffman_infer.huffman_encode.default(data, LUT, output, output_lengths)


def huffman_decode(
    A_rem: Tensor, A_exp: Tensor, Y: Tensor,
    offsets: Tensor,
    LUT1: Tensor, LUT2: Tensor, LUT3: Tensor, LUT4: Tensor,
    code_lengths: Tensor,
) -> None:
    torch.ops.bf16_huffman_infer.huffman_decode.default(
        A_rem, A_exp, Y, offsets, LUT1, LUT2, LUT3, LUT4, code_lengths)


def gemv_bf16_ans(A_rem: Tensor, A_exp: Tensor, X: Tensor, Y: Tensor, offsets: Tensor, LUT: Tensor) -> None:
    torch.ops.bf16_huffman_infer.gemv_bf16_ans.default(A_rem, A_exp, X, Y, offsets, LUT)


def ans_encode(data: Tensor, freq: Tensor, cum: Tensor, output: Tensor, output_lengths: Tensor) -> None:
    torch.ops.bf16_huffman_infer.ans_encode.default(data, freq, cum, output, output_lengths)


def ans_decode(A_rem: Tensor, A_exp: Tensor, Y: Tensor, offsets: Tensor, LUT: Tensor) -> None:
    torch.ops.bf16_huffman_infer.ans_decode.default(A_rem, A_exp, Y, offsets, LUT)


def encode_capacity(n_steps: int) -> int:
    """Words to reserve per task row of ``huffman_encode``'s output."""
    return int(_lib.load().bhi_encode_capacity(n_steps))


def ans_encode_capacity(n_steps: int) -> int:
    return int(_lib.load().bhi_ans_encode_capacity(n_steps))


def gemv_bf16_nibble(A_rem: Tensor, A_exp: Tensor, X: Tensor, Y: Tensor, offsets: Tensor, LUT: Tensor) -> None:
    torch.ops.bf16_huffman_infer_amd.gemv_bf16_nibble.default(A_rem, A_exp, X, Y, offsets, LUT)


def nibble_encode(data: Tensor, LUT: Tensor, output: Tensor, output_lengths: Tensor) -> None:
    torch.ops.bf16_huffman_infer_amd.nibble_encode.default(data, LUT, output, output_lengths)


def nibble_decode(A_rem: Tensor, A_exp: Tensor, Y: Tensor, offsets: Tensor, LUT: Tensor) -> None:
    torch.ops.bf16_huffman_infer_amd.nibble_decode.default(A_rem, A_exp, Y, offsets, LUT)


X_PLAIN, X_RMS, X_SILU_MUL = 0, 1, 2
X_TRANSFORM_MAX_ROWS = 4


def gemv_bf16_grouped(weights, X: Tensor, Ys, biases=None, residuals=None, x_mode: int = X_PLAIN, x_aux=None,
                      eps: float = 0.0) -> None:
    """One launch for up to four compressed weights that multiply the same ``X``.

    ``weights`` are weight modules of ONE class (:class:`HuffmanWeight`, :class:`ANSWeight`
    or :class:`NibbleWeight`: anything with ``rem, exp, offsets`` and ``LUT1, code_lengths``
    or ``LUT``) with equal ``split_k`` and ``Ks``; ``X`` is bf16 ``[batch, split_k, Ks]``,
    ``Ys[i]`` bf16 ``[batch, M_i]`` is written; ``biases[i]`` (bf16 ``[M_i]`` or None) is added
    as the reference's separate ``output += bias`` would (``functional.py:403-404``), then
    ``residuals[i]`` (bf16 ``[batch, M_i]`` or None) as a separate BF16 addition would.
    ``x_mode`` makes the kernel multiply with a function of ``X`` (batch <= 4, Huffman and
    rANS): ``X_RMS`` -- RMSNorm of ``X`` with ``x_aux`` = gamma bf16 ``[split_k*Ks]`` and
    ``eps``; ``X_SILU_MUL`` -- ``silu(x_aux) * X`` with ``x_aux`` = gate, shaped like ``X``.
    Not an op of the reference: it stands in for its q/k/v streams
    (``cudastream_utils.py:8-47``).  Plain function, not registered with the dispatcher; like
    the ops it only enqueues on the current stream.
    """
    if not 1 <= len(weights) <= 4 or len(weights) != len(Ys):
        raise RuntimeError("a group has 1 to 4 weights and one output per weight")
    first = weights[0]
    huffman = hasattr(first, "LUT1")
    if huffman:
        entry = "gemv_bf16_huffman_grouped"
    elif int(getattr(first, "MAGIC", 0)) != 0:
        entry = "gemv_bf16_nibble_grouped"
    else:
        entry = "gemv_bf16_ans_grouped"
    split_k, _, Ks = _weight_dims(first.rem, first.offsets)
    if X.dim() != 3 or X.shape[1] != split_k or X.shape[2] != Ks:
        raise RuntimeError(f"X must be [batch, {split_k}, {Ks}], got {tuple(X.shape)}")
    x_ptr = _req(X, torch.bfloat16, "X", first.rem)
    batch = X.shape[0]
    members = (_lib.GemvMember * len(weights))()
    if biases is None:
        biases = [None] * len(weights)
    if residuals is None:
        residuals = [None] * len(weights)
    for m, w, Y, b, r in zip(members, weights, Ys, biases, residuals):
        if type(w) is not type(first):
            raise RuntimeError("the weights of a group must use one codec")
        sk, M, ks = _weight_dims(w.rem, w.offsets)
        if (sk, ks) != (split_k, Ks):
            raise RuntimeError("the weights of a group must share split_k and Ks")
        if tuple(Y.shape) != (batch, M):
            raise RuntimeError(f"Y must be [{batch}, {M}], got {tuple(Y.shape)}")
        _fill_member(m, w, Y, b, first.rem)
        if r is not None:
            if tuple(r.shape) != (batch, M):
                raise RuntimeError(f"residual must be [{batch}, {M}], got {tuple(r.shape)}")
            m.residual = _req(r, torch.bfloat16, "residual", first.rem)
    lib = _lib.load()
    with torch.cuda.device(first.rem.device):
        if x_mode == X_PLAIN:
            rc = getattr(lib, "bhi_" + entry)(members, len(weights), x_ptr, split_k, Ks, batch, _stream(first.rem))
        else:
            if entry == "gemv_bf16_nibble_grouped":
                raise RuntimeError("the nibble codec's kernels take X as it is")
            want = (split_k * Ks,) if x_mode == X_RMS else (batch, split_k * Ks)
            if x_aux is None or x_aux.numel() != want[-1] * (1 if x_mode == X_RMS else batch):
                raise RuntimeError(f"x_aux must hold {want} values")
            entry += "_x"
            rc = getattr(lib, "bhi_" + entry)(members, len(weights), x_ptr, split_k, Ks, batch, int(x_mode),
                                              _req(x_aux, torch.bfloat16, "x_aux", first.rem), float(eps), _stream(first.rem))
    _lib.check(rc, entry)


def rms_norm(x: Tensor, gamma: Tensor, eps: float) -> Tensor:
    """``bf16(x * rsqrt(mean(x^2) + eps) * gamma)`` over the last dimension, one rounding: the
    arithmetic (reduction order included) of the RMSNorm that :func:`gemv_bf16_grouped` fuses."""
    lib = _lib.load()
    K = x.shape[-1]
    flat = x.reshape(-1, K).contiguous()
    out = torch.empty_like(flat)
    g = _req(gamma.contiguous(), torch.bfloat16, "gamma", flat)
    with torch.cuda.device(flat.device):
        for r0 in range(0, flat.shape[0], X_TRANSFORM_MAX_ROWS):
            rows = flat[r0:r0 + X_TRANSFORM_MAX_ROWS]
            _lib.check(lib.bhi_rms_norm(_req(rows, torch.bfloat16, "x"), g, out[r0:].data_ptr(), rows.shape[0], K, float(eps),
                                        _stream(flat)), "rms_norm")
    return out.view(x.shape)


def silu_mul(gate: Tensor, up: Tensor) -> Tensor:
    """``bf16(bf16(silu(gate)) * up)``: the roundings of a BF16 ``F.silu(gate) * up``, as the GEMV
    fuses them."""
    if gate.shape != up.shape:
        raise RuntimeError("gate and up must have one shape")
    g, u = gate.contiguous(), up.contiguous()
    out = torch.empty_like(g)
    with torch.cuda.device(g.device):
        _lib.check(_lib.load().bhi_silu_mul(_req(g, torch.bfloat16, "gate"), _req(u, torch.bfloat16, "up", g), out.data_ptr(),
                                            g.numel(), _stream(g)), "silu_mul")
    return out


def decode_attention(qk: Tensor, v: Tensor, norm_weight, cos: Tensor, sin: Tensor, pos: Tensor, k_cache: Tensor,
                     v_cache: Tensor, out: Tensor = None, eps: float = 1e-6, scale: float = None) -> Tensor:
    """The attention step of one new token of a decoder layer in one launch (no counterpart in the
    reference, which leaves attention to the model code): per-head RMSNorm (times ``norm_weight``,
    bf16 ``[q_heads + kv_heads, 128]`` or None) and rotation of the projected heads ``qk`` (bf16
    ``[q_heads + kv_heads, 128]``, q heads first) by row ``pos`` of ``cos`` / ``sin`` (fp32
    ``[max_len, 128]``, ``out = x * cos + swap_halves(x) * sin``), ``k`` and ``v`` (bf16 ``[kv_heads, 128]``)
    written into slot ``pos`` of ``k_cache`` / ``v_cache`` (bf16 ``[kv_heads, max_len, 128]``), and
    ``softmax(q k^T * scale) v`` over slots ``0..pos`` per q head.  ``pos`` is an int64 tensor of one
    element ON THE DEVICE: a recorded graph reads it at every replay.  Returns ``out`` (bf16
    ``[q_heads, 128]``)."""
    heads, d = qk.shape
    kv_heads, max_len, _ = k_cache.shape
    q_heads = heads - kv_heads
    if tuple(v.shape) != (kv_heads, d) or tuple(v_cache.shape) != (kv_heads, max_len, d):
        raise RuntimeError("v must be [kv_heads, head_dim] and the caches [kv_heads, max_len, head_dim]")
    if tuple(cos.shape) != (max_len, d) or tuple(sin.shape) != (max_len, d):
        raise RuntimeError(f"cos and sin must be [{max_len}, {d}]")
    if pos.numel() != 1 or pos.dtype != torch.int64 or pos.device != qk.device:
        raise RuntimeError("pos must be one int64 on the device of qk")
    if norm_weight is not None and tuple(norm_weight.shape) != (heads, d):
        raise RuntimeError(f"norm_weight must be [{heads}, {d}]")
    if out is None:
        out = torch.empty((q_heads, d), dtype=torch.bfloat16, device=qk.device)
    elif tuple(out.shape) != (q_heads, d):
        raise RuntimeError(f"out must be [{q_heads}, {d}]")
    lib = _lib.load()
    with torch.cuda.device(qk.device):
        rc = lib.bhi_decode_attention(
            _req(qk, torch.bfloat16, "qk"), _req(v, torch.bfloat16, "v", qk),
            None if norm_weight is None else _req(norm_weight, torch.bfloat16, "norm_weight", qk),
            _req(cos, torch.float32, "cos", qk), _req(sin, torch.float32, "sin", qk), pos.data_ptr(),
            _req(k_cache, torch.bfloat16, "k_cache", qk), _req(v_cache, torch.bfloat16, "v_cache", qk),
            _req(out, torch.bfloat16, "out", qk), q_heads, kv_heads, d, max_len, float(eps),
            float(d ** -0.5 if scale is None else scale), _stream(qk))
    _lib.check(rc, "decode_attention")
    return out


def _fill_member(m, w, Y: Tensor, bias, ref: Tensor) -> bool:
    """Fills one ``bhi_gemv_member`` from a weight module; returns whether it is a Huffman weight."""
    huffman = hasattr(w, "LUT1")
    _, M, _ = _weight_dims(w.rem, w.offsets)
    m.A_rem = _req(w.rem, torch.uint8, "A_rem", ref)
    m.A_exp = _req(w.exp, torch.int32, "A_exp", ref)
    m.exp_words = w.exp.numel()
    m.Y = _req(Y, torch.bfloat16, "Y", ref)
    m.offsets = _req(w.offsets, torch.int32, "offsets", ref)
    if huffman:
        m.table = _req(w.LUT1, torch.uint8, "LUT1", ref)
        m.table_bytes = w.LUT1.numel()
        m.header = _req(w.code_lengths, torch.uint8, "code_lengths", ref)
    else:
        m.table = _req(w.LUT, torch.int32, "LUT", ref)
        m.table_bytes = w.LUT.numel() * 4
        m.header = None
    m.M = M
    if bias is not None:
        if tuple(bias.shape) != (M,):
            raise RuntimeError(f"bias must be [{M}], got {tuple(bias.shape)}")
        m.bias = _req(bias, torch.bfloat16, "bias", ref)
    return huffman


GEMM_MAX_ROWS = 32
_workspaces = {}          # (device, stream) -> [zero-initialised uint8 tensors]; every launch leaves its counters at zero


def _gemm_workspace(device: torch.device, stream: int, nbytes: int, allocate=None) -> Tensor:
    """The fused matrix product's workspace for launches on ``stream`` of ``device``: partial
    sums of K slices and the arrival counters of their row blocks.  One per (device, stream):
    launches on one stream run one after the other and may share it, launches on different
    streams may overlap and must not.  Grown by replacement; the old one is kept alive because
    enqueued launches may still use it."""
    key = (device, stream)
    held = _workspaces.get(key)
    if held is None or held[-1].numel() < nbytes:
        make = allocate or (lambda n: torch.zeros(n, dtype=torch.uint8, device=device))
        _workspaces[key] = (held or []) + [make(max(nbytes, 1 << 20))]
        held = _workspaces[key]
    return held[-1]


def gemm_bf16(weight, X: Tensor, Y: Tensor, bias=None, static_workspace: bool = False, residual=None) -> None:
    """``Y = X @ W.T (+ bias)`` for up to 32 rows of ``X`` with ``W`` held compressed
    (:class:`HuffmanWeight` or :class:`ANSWeight`), decoded inside the matrix-core kernel.

    Takes the place of ``get_weight()`` + ``F.linear`` in the reference's path above eight
    rows (``functional.py:405-407, 460-462``).  ``X`` bf16 ``[rows, split_k, Ks]``, ``Y`` bf16
    ``[rows, M]`` written; ``bias`` (bf16 ``[M]``) and then ``residual`` (bf16 ``[rows, M]``) are added
    as separate BF16 additions would.  Plain function: only enqueues on the current stream.  Products that
    are cut along K keep their partial sums in a workspace that belongs to the (device, stream)
    pair of the call and is allocated (and zeroed by a fill kernel) at the first such call on
    that stream -- also under stream capture, where the allocation comes from the graph's own
    pool and the fill becomes a node in front of the product.  ``static_workspace=True`` (Huffman
    weights) allocates nothing and uses the array built into the library instead: ONE array per
    GPU, so launches that take it and may overlap on the GPU (different streams) race."""
    lib = _lib.load()
    split_k, M, Ks = _weight_dims(weight.rem, weight.offsets)
    if X.dim() != 3 or X.shape[1] != split_k or X.shape[2] != Ks:
        raise RuntimeError(f"X must be [rows, {split_k}, {Ks}], got {tuple(X.shape)}")
    rows = X.shape[0]
    if tuple(Y.shape) != (rows, M):
        raise RuntimeError(f"Y must be [{rows}, {M}], got {tuple(Y.shape)}")
    member = (_lib.GemvMember * 1)()
    x_ptr = _req(X, torch.bfloat16, "X", weight.rem)
    huffman = _fill_member(member[0], weight, Y, bias, weight.rem)
    if residual is not None:
        if tuple(residual.shape) != (rows, M):
            raise RuntimeError(f"residual must be [{rows}, {M}], got {tuple(residual.shape)}")
        member[0].residual = _req(residual, torch.bfloat16, "residual", weight.rem)
    name = "gemm_bf16_huffman" if huffman else "gemm_bf16_ans"
    device = weight.rem.device
    stream = _stream(weight.rem)
    with torch.cuda.device(device):
        need = int(lib.bhi_gemm_workspace_bytes(split_k, M, Ks, rows))
        if need < 0:
            _lib.check(need, name)
        ws = None
        if need == 0:
            rc = getattr(lib, "bhi_" + name)(member, x_ptr, split_k, Ks, rows, None, 0, stream)
        elif static_workspace:
            if not huffman:
                raise RuntimeError("gemm_bf16: the built-in workspace serves Huffman weights only")
            if device not in _ready_devices:
                raise RuntimeError("gemm_bf16: the library has not been used on this device outside a stream capture yet")
            rc = lib.bhi_gemm_bf16_huffman_static(member, x_ptr, split_k, Ks, rows, stream)
        else:
            ws = _gemm_workspace(device, stream, need)
            rc = getattr(lib, "bhi_" + name)(member, x_ptr, split_k, Ks, rows, ws.data_ptr(), ws.numel(), stream)
        if rc != 0 and ws is not None:
            # the launch did not happen or was cut short: its counters may not be zero any more
            lib.bhi_gemm_workspace_reset(ws.data_ptr(), ws.numel(), stream)
    _lib.check(rc, name)


def gemm_bf16_grouped(weights, X: Tensor, Ys, biases=None, residuals=None) -> None:
    """:func:`gemm_bf16` for up to four weights of one class (Huffman or rANS) and one ``split_k`` / ``Ks``
    that multiply the same ``X``: one grid when their rows together are enough for the kernel to
    run without cutting along K (8192 rows), else one launch per member.  Stands in, like
    :func:`gemv_bf16_grouped`, for the reference's parallel streams (``cudastream_utils.py:8-47``)."""
    n = len(weights)
    if not 1 <= n <= 4 or n != len(Ys):
        raise RuntimeError("a group has 1 to 4 weights and one output per weight")
    biases = [None] * n if biases is None else list(biases)
    residuals = [None] * n if residuals is None else list(residuals)
    first = weights[0]
    split_k, _, Ks = _weight_dims(first.rem, first.offsets)
    if X.dim() != 3 or X.shape[1] != split_k or X.shape[2] != Ks:
        raise RuntimeError(f"X must be [rows, {split_k}, {Ks}], got {tuple(X.shape)}")
    rows = X.shape[0]
    dims = [_weight_dims(w.rem, w.offsets) for w in weights]
    if any(type(w) is not type(first) for w in weights):
        raise RuntimeError("the weights of a group must use one codec")
    if any((sk, ks) != (split_k, Ks) for sk, _, ks in dims):
        raise RuntimeError("the weights of a group must share split_k and Ks")
    lib = _lib.load()
    total = sum(M for _, M, _ in dims)
    if n == 1 or int(lib.bhi_gemm_workspace_bytes(split_k, total, Ks, rows)) != 0:
        for w, Y, b, r in zip(weights, Ys, biases, residuals):
            gemm_bf16(w, X, Y, b, residual=r)
        return
    members = (_lib.GemvMember * n)()
    x_ptr = _req(X, torch.bfloat16, "X", first.rem)
    huffman = True
    for m, w, (_, M, _), Y, b, r in zip(members, weights, dims, Ys, biases, residuals):
        if tuple(Y.shape) != (rows, M):
            raise RuntimeError(f"Y must be [{rows}, {M}], got {tuple(Y.shape)}")
        huffman = _fill_member(m, w, Y, b, first.rem)
        if r is not None:
            if tuple(r.shape) != (rows, M):
                raise RuntimeError(f"residual must be [{rows}, {M}], got {tuple(r.shape)}")
            m.residual = _req(r, torch.bfloat16, "residual", first.rem)
    name = "gemm_bf16_huffman_grouped" if huffman else "gemm_bf16_ans_grouped"
    with torch.cuda.device(first.rem.device):
        rc = getattr(lib, "bhi_" + name)(members, n, x_ptr, split_k, Ks, rows, _stream(first.rem))
    _lib.check(rc, name)


def nibble_encode_capacity(n_steps: int) -> int:
    return int(_lib.load().bhi_nibble_encode_capacity(n_steps))

"""Sequence-mixing ops of hybrid (windowed attention + linear recurrence)
models: dispatch between the gfx950 kernels of ``csrc/seqmix.hip`` and the
torch references in ``ops.ref`` (CPU execution and numerics oracle).

The kernels live in their own small shared library ``_nxdi_seqmix.so`` with
a C ABI, loaded through ctypes: it has no torch headers, so a fresh checkout
compiles it with one ``hipcc`` call in seconds and a model that needs only
these ops never waits for the large extension. Launches go to torch's
current HIP stream. On a GPU tensor the library is required — there is no
silent fallback.
"""

from __future__ import annotations

import ctypes
import os
import subprocess
import threading
from typing import Optional

import torch

from neuronx_distributed_inference_amd.ops import ref

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "_nxdi_seqmix.so")
SRC_PATH = os.path.join(_HERE, "csrc", "seqmix.hip")
HIPCC_FLAGS = [
    "-O3", "-std=c++17", "--offload-arch=gfx950", "-shared", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]

_lib = None
_lib_error: Optional[BaseException] = None
_lock = threading.Lock()


def _compile(dst: str) -> str:
    hipcc = os.environ.get("HIPCC") or (
        "/opt/rocm/bin/hipcc" if os.path.exists("/opt/rocm/bin/hipcc") else "hipcc")
    tmp = dst + ".%d.tmp" % os.getpid()
    try:
        subprocess.run([hipcc] + HIPCC_FLAGS + ["-o", tmp, SRC_PATH], check=True,
                       stdout=subprocess.DEVNULL, stderr=subprocess.PIPE)
        os.replace(tmp, dst)
    finally:
        if os.path.exists(tmp):
            os.unlink(tmp)
    return dst


def build(force: bool = False) -> str:
    """Compile the library in-tree (cross-compiles without a GPU). When the
    package directory is read-only the library goes to the user's temp
    directory, named after the source's modification time."""
    global LIB_PATH
    if not force and os.path.exists(LIB_PATH) and \
            os.path.getmtime(LIB_PATH) >= os.path.getmtime(SRC_PATH):
        return LIB_PATH
    try:
        return _compile(LIB_PATH)
    except (OSError, subprocess.CalledProcessError):
        if os.access(os.path.dirname(LIB_PATH), os.W_OK):
            raise                      # a real compile error, not a read-only tree
        import tempfile

        alt = os.path.join(tempfile.gettempdir(), "nxdi_seqmix_%d_%d.so" % (
            os.getuid(), int(os.path.getmtime(SRC_PATH))))
        if force or not os.path.exists(alt):
            _compile(alt)
        LIB_PATH = alt
        return LIB_PATH


def _load():
    global _lib, _lib_error
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        try:
            build()
            _lib = ctypes.CDLL(LIB_PATH)
        except BaseException as e:  # noqa: BLE001
            _lib_error = e
            raise RuntimeError(
                "sequence-mixing op called on a GPU tensor but _nxdi_seqmix.so "
                f"could not be built/loaded: {e!r}") from e
    return _lib


def library_available() -> bool:
    try:
        _load()
        return True
    except RuntimeError:
        return False


def _p(t: Optional[torch.Tensor]):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _is_bf16(t: torch.Tensor) -> int:
    if t.dtype == torch.bfloat16:
        return 1
    if t.dtype == torch.float32:
        return 0
    raise TypeError(f"seqmix ops take float32 or bfloat16, got {t.dtype}")


def _check(rc: int, name: str):
    if rc != 0:
        raise RuntimeError(f"{name}: launch failed / unsupported shape (code {rc})")


def _i32(t: torch.Tensor) -> torch.Tensor:
    return t if t.dtype == torch.int32 and t.is_contiguous() else t.to(torch.int32).contiguous()


def _f32(t: torch.Tensor) -> torch.Tensor:
    return t if t.dtype == torch.float32 and t.is_contiguous() else t.float().contiguous()


def _rows_view(t: torch.Tensor):
    """(..., C) tensor whose leading dims collapse to rows with one stride
    (a column slice of a fused GEMM output qualifies): returns row stride."""
    assert t.stride(-1) == 1, "innermost dim must be contiguous"
    if t.dim() == 3:
        return _token_stride(t)
    return t.stride(0)


def _token_stride(t: torch.Tensor) -> int:
    """Stride between consecutive tokens of a (B, S, ...) tensor whose
    tokens are uniformly strided (a size-1 axis has no stride of its own)."""
    B, S = t.shape[0], t.shape[1]
    if S == 1:
        return t.stride(0) if B > 1 else max(t.stride(0), t.stride(1))
    assert B == 1 or t.stride(0) == t.stride(1) * S, "rows must be uniformly strided"
    return t.stride(1)


class StepLayout:
    """Per-step ragged-batch descriptors shared by every layer's kernels:
    int32 positions (B,S), state slots (B,), valid-token counts (B,)."""

    def __init__(self, positions: torch.Tensor, seq_ids: torch.Tensor):
        self.positions = _i32(positions)
        self.seq_ids = _i32(seq_ids)
        self.nvalid = (self.positions >= 0).sum(-1).to(torch.int32)
        self._i32 = {}
        # the residual stream in the GEMM input dtype, handed from one
        # sublayer's residual kernel to the next sublayer (None: not yet made)
        self.stream_copy = None
        # True when every row of the step starts its sequence (a whole prompt)
        self.fresh = False

    def i32(self, t: torch.Tensor) -> torch.Tensor:
        """int32 copy of a per-step index tensor (block table, slot mapping),
        converted once per step instead of once per layer."""
        key = (t.data_ptr(), tuple(t.shape), t.dtype)
        hit = self._i32.get(key)
        if hit is None:
            hit = self._i32[key] = (t, _i32(t))      # keeps `t` alive: the pointer stays its
        return hit[1]


# ----------------------------------------------------------------------
def layer_norm(x, weight, eps: float, out_dtype: torch.dtype):
    """Bias-free LayerNorm of an fp32 stream, fp32 statistics."""
    if x.is_cuda:
        lib = _load()
        x = _f32(x)
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        C = x.shape[-1]
        _check(lib.nx_layer_norm(_p(x), _p(_f32(weight)), _p(out), _is_bf16(out),
                                 ctypes.c_long(x.numel() // C), C,
                                 ctypes.c_float(eps), _stream()), "layer_norm")
        return out
    return ref.layer_norm(x, weight, eps, out_dtype)


def short_conv(x, w, tail, step: StepLayout, activation: str = "none",
               residual: bool = False, out_dtype=torch.float32, bias=None):
    """Depthwise causal conv over time with a carried tail and an optional
    per-channel bias (see ref.short_conv). Does not advance the tail: call
    short_conv_commit."""
    if x.is_cuda:
        lib = _load()
        B, S, C = x.shape
        y = torch.empty(B, S, C, dtype=out_dtype, device=x.device)
        _check(lib.nx_short_conv(
            _p(x), ctypes.c_long(_rows_view(x)), _is_bf16(x), _p(_f32(w)), _p(tail), _p(step.positions),
            _p(step.seq_ids), _p(step.nvalid), _p(y), _is_bf16(y), B, S, C, w.shape[1],
            int(activation == "silu"), int(residual),
            _p(None if bias is None else _f32(bias)), _stream()), "short_conv")
        return y
    return ref.short_conv(x, w, tail, step.positions, step.seq_ids,
                          activation, residual, out_dtype, bias)


def short_conv_commit(x, tail, step: StepLayout):
    if x.is_cuda:
        lib = _load()
        B, S, C = x.shape
        assert tail.dtype == torch.float32 and tail.is_contiguous()
        _check(lib.nx_short_conv_commit(
            _p(x), ctypes.c_long(_rows_view(x)), _is_bf16(x), _p(tail), _p(step.positions), _p(step.seq_ids),
            _p(step.nvalid), B, S, C, tail.shape[1], _stream()), "short_conv_commit")
        return
    ref.short_conv_commit(x, tail, step.positions, step.seq_ids)


def paged_kv_write(k_cache, v_cache, k_new, v_new, slot_mapping, step: "StepLayout" = None):
    """Scatter k_new (N, G*Dk) / v_new (N, G*Dv) rows (row-strided views
    allowed) into paged caches (blocks, block, G, D*). ``v_cache``/``v_new``
    may be None for caches whose values live inside the key rows."""
    if k_cache.is_cuda:
        lib = _load()
        N = k_new.shape[0]
        GDk = k_cache.shape[2] * k_cache.shape[3]
        GDv = 0 if v_cache is None else v_cache.shape[2] * v_cache.shape[3]
        assert k_new.shape[1] == GDk and k_new.dtype == k_cache.dtype and k_new.stride(1) == 1
        assert k_cache.is_contiguous()
        if v_cache is not None:
            assert v_new.shape[1] == GDv and v_new.dtype == v_cache.dtype == k_cache.dtype
            assert v_new.stride(1) == 1 and v_cache.is_contiguous()
        _check(lib.nx_paged_kv_write(
            _p(k_cache), _p(v_cache), _p(k_new), ctypes.c_long(k_new.stride(0)),
            _p(v_new), ctypes.c_long(0 if v_new is None else v_new.stride(0)),
            _is_bf16(k_cache),
            _p(_i32(slot_mapping) if step is None else step.i32(slot_mapping)),
            ctypes.c_long(N), GDk, GDv,
            ctypes.c_long(k_cache.shape[0] * k_cache.shape[1]), _stream()),
            "paged_kv_write")
        return
    G = k_cache.shape[2]
    ref.paged_kv_write(k_cache, v_cache, k_new.reshape(k_new.shape[0], G, -1),
                       None if v_new is None else v_new.reshape(v_new.shape[0], G, -1),
                       slot_mapping)


def paged_attention(q, k_cache, v_cache, step: StepLayout, block_table, scale: float,
                    num_heads: int, window: Optional[int] = None, keep_first: int = 0,
                    r1=None, r2=None, gate=None, softcap: float = 0.0, sink=None,
                    q_temp=None, out_dtype=None, gate_per_head: bool = False,
                    chunk: int = 0, slopes=None):
    """q (B,S,H*Dk) (row-strided view allowed) against the paged cache ->
    (B,S,H*Dv). Options (see ref.paged_attention): sliding ``window`` with
    ``keep_first`` always-visible tokens (None = plain causal), ``chunk`` > 0
    = only keys of the query's own block of that many positions, log-distance
    penalty ``r1``/``r2`` or linear distance penalty ``slopes`` (H,), tanh
    score cap, per-head softmax ``sink``, query
    temperature ``q_temp`` = (coef, every), sigmoid output ``gate``
    ((B,S,H*Dv), or (B,S,H) with ``gate_per_head``).
    ``v_cache`` may be ``k_cache[..., :Dv]`` (values inside the key rows)."""
    B, S = q.shape[0], q.shape[1]
    H = num_heads
    G, Dk = k_cache.shape[2], k_cache.shape[3]
    Dv = v_cache.shape[3]
    out_dtype = out_dtype or q.dtype
    assert slopes is None or r1 is None, "one distance penalty at a time"
    if q.is_cuda:
        lib = _load()
        out = torch.empty(B, S, H * Dv, dtype=out_dtype, device=q.device)
        bt = step.i32(block_table)
        if slopes is not None:
            r1, r2 = slopes, None          # the kernels read a lone r1 as slopes
        assert k_cache.stride(3) == 1 and v_cache.stride(3) == 1
        assert k_cache.stride(1) == k_cache.stride(2) * G and v_cache.stride(1) == v_cache.stride(2) * G
        assert k_cache.stride(0) == k_cache.stride(1) * k_cache.shape[1]
        assert v_cache.stride(0) == v_cache.stride(1) * v_cache.shape[1]
        assert k_cache.dtype == v_cache.dtype == q.dtype
        coef, every = (0.0, 0) if q_temp is None else (float(q_temp[0]), int(q_temp[1]))
        # single-token steps over latent caches (values inside the one key
        # row): few workgroups per step, so the keys are split over several
        # and merged; the partials need a workspace
        ws, nks = None, 1
        if S == 1 and G == 1 and q.dtype == torch.bfloat16 and \
                v_cache.data_ptr() == k_cache.data_ptr():
            groups = B * ((H + 15) // 16) * ((Dv + 511) // 512)
            span = bt.shape[1] * k_cache.shape[1]           # most keys a token can see
            if window is not None:
                span = min(span, int(window) + 31)
            if chunk:
                span = min(span, int(chunk) + 31)
            nks = max(1, min(8, 256 // max(groups, 1), span // 128))
            if nks > 1:
                ws = torch.empty(B * H * nks * (Dv + 2), dtype=torch.float32, device=q.device)
        _check(lib.nx_paged_attn(
            _p(q), ctypes.c_long(_rows_view(q)), _p(k_cache), ctypes.c_long(k_cache.stride(1)),
            ctypes.c_long(k_cache.stride(2)), _p(v_cache), ctypes.c_long(v_cache.stride(1)),
            ctypes.c_long(v_cache.stride(2)),
            _p(step.positions), _p(step.seq_ids), _p(bt), bt.shape[1],
            _p(None if r1 is None else _f32(r1)), _p(None if r2 is None else _f32(r2)),
            _p(None if sink is None else _f32(sink)),
            _p(gate), ctypes.c_long(0 if gate is None else _rows_view(gate)),
            _p(out), _is_bf16(q), _is_bf16(out), B, S, H, G, Dk, Dv,
            k_cache.shape[1], ctypes.c_float(scale),
            int(window) if window is not None else 0x7fffffff, int(keep_first),
            ctypes.c_float(softcap or 0.0), ctypes.c_float(coef), every,
            _p(ws), nks, int(bool(gate_per_head)), int(chunk or 0), _stream()),
            "paged_attention")
        return out
    return ref.paged_attention(
        q.reshape(B, S, H, Dk), k_cache, v_cache, step.positions, block_table, scale,
        window=window, keep_first=keep_first, r1=r1, r2=r2, gate=gate,
        softcap=softcap or 0.0, sink=sink, q_temp=q_temp, out_dtype=out_dtype,
        gate_per_head=gate_per_head, chunk=int(chunk or 0), slopes=slopes)


def window_bias_attention(q, k_cache, v_cache, step: StepLayout, block_table,
                          r1, r2, scale: float, window: int, keep_first: int,
                          num_heads: int, gate=None, out_dtype=None):
    """Sliding window + kept first tokens with a log-distance penalty."""
    return paged_attention(q, k_cache, v_cache, step, block_table, scale, num_heads,
                           window=window, keep_first=keep_first, r1=r1, r2=r2,
                           gate=gate, out_dtype=out_dtype)


def gated_delta_rule(qkv, beta, a, dt_bias, a_log, gate, norm_w, eps: float,
                     state, step: StepLayout, kv_heads: int, dim: int, vdim: int,
                     out_dtype=torch.float32, gate_act: str = "sigmoid"):
    """Gated delta-rule recurrence over the step's tokens, state carried in
    `state` (slots, H, vdim, dim) fp32; see ref.gated_delta_rule. ``a`` is
    (B,S,H*dim) for a decay per key channel or (B,S,H) for one per head."""
    assert gate_act in ("sigmoid", "silu")
    if qkv.is_cuda:
        lib = _load()
        B, S = qkv.shape[0], qkv.shape[1]
        H = beta.shape[-1]
        per_head = a.shape[-1] == H and dim != 1
        assert a.shape[-1] == (H if per_head else H * dim)
        assert dt_bias.numel() == a.shape[-1]
        assert qkv.dtype == torch.float32 and state.dtype == torch.float32
        assert beta.dtype == a.dtype == gate.dtype == out_dtype
        out = torch.empty(B, S, H * vdim, dtype=out_dtype, device=qkv.device)
        obuf = torch.empty(B, S, H * vdim, dtype=torch.float32, device=qkv.device)
        PS = (2 * kv_heads + H) * dim + H + kv_heads
        prep = torch.empty(B, S, PS, dtype=torch.float32, device=qkv.device)
        _check(lib.nx_gated_delta(
            _p(qkv), ctypes.c_long(_rows_view(qkv)), _p(beta),
            ctypes.c_long(_rows_view(beta)), _p(a), ctypes.c_long(_rows_view(a)),
            _p(gate), ctypes.c_long(_rows_view(gate)), _p(_f32(dt_bias)),
            _p(_f32(a_log)), _p(_f32(norm_w)), ctypes.c_float(eps), _p(state),
            _p(step.positions), _p(step.seq_ids), _p(step.nvalid), _p(prep),
            ctypes.c_long(PS), _p(obuf), _p(out),
            _is_bf16(beta), B, S, H, kv_heads, dim, vdim, int(per_head),
            int(gate_act == "silu"), _stream()),
            "gated_delta_rule")
        return out
    return ref.gated_delta_rule(qkv, beta, a, dt_bias, a_log, gate, norm_w, eps,
                                state, step.positions, step.seq_ids, kv_heads,
                                dim, vdim, out_dtype, gate_act)


def softcap(logits, cap: float):
    """cap * tanh(logits / cap) in fp32."""
    if logits.is_cuda:
        lib = _load()
        x = logits.contiguous()
        out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
        _check(lib.nx_softcap(_p(x), _is_bf16(x), _p(out), ctypes.c_long(x.numel()),
                              ctypes.c_float(cap), _stream()), "softcap")
        return out
    return ref.softcap(logits, cap)


def residual_add(x, a, sa: float = 1.0, b=None, sb: float = 1.0):
    """In place on the fp32 stream: x += sa*a (+ sb*b)."""
    if x.is_cuda:
        lib = _load()
        assert x.dtype == torch.float32 and x.is_contiguous()
        a = a.contiguous()
        if b is not None:
            b = b.contiguous()
            assert b.dtype == a.dtype
        _check(lib.nx_residual_add(_p(x), _p(a), ctypes.c_float(sa), _p(b),
                                   ctypes.c_float(sb), _is_bf16(a),
                                   ctypes.c_long(x.numel()), _stream()), "residual_add")
        return x
    x.add_(a.float(), alpha=sa)
    if b is not None:
        x.add_(b.float(), alpha=sb)
    return x


def gelu_tanh_mul_fused(gate_up):
    """(rows, 2I) [gate | up] -> gelu_tanh(gate) * up."""
    I = gate_up.shape[-1] // 2
    if gate_up.is_cuda:
        lib = _load()
        gu = gate_up.contiguous()
        out = torch.empty(gu.shape[:-1] + (I,), dtype=gu.dtype, device=gu.device)
        _check(lib.nx_gelu_mul(_p(gu), _p(out), _is_bf16(gu),
                               ctypes.c_long(gu.numel() // (2 * I)), I, _stream()),
               "gelu_tanh_mul_fused")
        return out
    g, u = gate_up.float().chunk(2, dim=-1)
    return ref.gelu_tanh_mul(g, u).to(gate_up.dtype)


def rms_norm(x, weight, eps: float, one_plus: bool = False, out_dtype=None, out=None):
    """RMS norm over the last axis with fp32 statistics: x / sqrt(mean(x^2)
    + eps) * w (or * (1 + w) for weights stored around zero). ``x`` may be a
    column slice of a wider tensor; ``out`` may be a column slice to fill."""
    out_dtype = out_dtype or (out.dtype if out is not None else x.dtype)
    if x.is_cuda:
        lib = _load()
        C = x.shape[-1]
        if out is None:
            out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        assert out.shape == x.shape and out.dtype == out_dtype
        rows = x.numel() // C
        _check(lib.nx_rms_norm(
            _p(x), ctypes.c_long(_rows_view(x)), _is_bf16(x), _p(_f32(weight)), int(one_plus),
            ctypes.c_float(eps), _p(out), ctypes.c_long(_rows_view(out)), _is_bf16(out),
            ctypes.c_long(rows), C, _stream()), "rms_norm")
        return out
    y = ref.rms_norm_rows(x, weight, eps, one_plus, out_dtype)
    if out is not None:
        out.copy_(y)
        return out
    return y


def add_rms_norm(stream, y, weight, eps: float, one_plus: bool = True, copy_dtype=None,
                 extra=None, coef=None, next_weight=None):
    """Post-norm residual step on the fp32 stream, in place:
    stream += rms_norm(y) * w (``one_plus``: * (1 + w)). With ``extra``
    (same shape as y) and ``coef`` (rows, n) fp32, the normed vector is
    y + sum(coef[row]) * extra[row] (experts that pass their input through).
    Returns the updated stream cast to ``copy_dtype`` (the next sublayer's
    GEMM input), or, with ``next_weight``, the next sublayer's pre-norm
    rms_norm(stream) * next_weight in ``copy_dtype``; None without a
    ``copy_dtype``."""
    assert (extra is None) == (coef is None)
    if stream.is_cuda:
        lib = _load()
        assert stream.dtype == torch.float32 and stream.is_contiguous()
        y = y.contiguous()
        C = stream.shape[-1]
        rows = stream.numel() // C
        copy = None
        if copy_dtype is not None and (copy_dtype != torch.float32 or next_weight is not None):
            copy = torch.empty(stream.shape, dtype=copy_dtype, device=stream.device)
        nc, cs = 0, 0
        if extra is not None:
            extra = extra.contiguous()
            assert extra.dtype == y.dtype and extra.numel() == y.numel()
            assert coef.dtype == torch.float32 and coef.stride(-1) == 1 and coef.dim() == 2
            assert coef.shape[0] == rows
            nc, cs = coef.shape[1], coef.stride(0)
        _check(lib.nx_add_rms_norm(
            _p(stream), _p(y), _is_bf16(y), _p(_f32(weight)), int(one_plus),
            ctypes.c_float(eps), _p(copy), 0 if copy is None else _is_bf16(copy),
            _p(extra), _p(coef), ctypes.c_long(cs), nc,
            _p(None if next_weight is None else _f32(next_weight)),
            ctypes.c_long(rows), C, _stream()), "add_rms_norm")
        if copy_dtype == torch.float32 and next_weight is None:
            return stream
        return copy
    v = y.float()
    if extra is not None:
        v = v + coef.float().sum(-1).view(*y.shape[:-1], 1) * extra.float()
    stream.add_(ref.rms_norm_rows(v, weight, eps, one_plus, torch.float32))
    if copy_dtype is None:
        return None
    if next_weight is not None:
        return ref.rms_norm_rows(stream, next_weight, eps, False, copy_dtype)
    return stream if copy_dtype == torch.float32 else stream.to(copy_dtype)


def rotate_interleaved(x, step: StepLayout, inv_freq, out=None, out_dtype=None):
    """Rotary positions on interleaved channel pairs (2i, 2i+1) of the first
    2*len(inv_freq) channels of every head; angles p * inv_freq[i] in fp32.
    x (B,S,N,C), possibly a strided view; ``out`` likewise (may be a slice of
    a wider buffer). Channels past the rotated ones are copied."""
    out_dtype = out_dtype or (out.dtype if out is not None else x.dtype)
    if x.is_cuda:
        lib = _load()
        B, S, N, C = x.shape
        if out is None:
            out = torch.empty(B, S, N, C, dtype=out_dtype, device=x.device)
        assert x.stride(3) == 1 and out.stride(3) == 1
        assert 2 * inv_freq.numel() <= C
        _check(lib.nx_rope_pairs(
            _p(x), ctypes.c_long(_token_stride(x)), ctypes.c_long(x.stride(2)), _is_bf16(x),
            _p(out), ctypes.c_long(_token_stride(out)), ctypes.c_long(out.stride(2)),
            _is_bf16(out),
            _p(step.positions), _p(_f32(inv_freq)), inv_freq.numel(),
            ctypes.c_long(B * S), N, C, _stream()), "rotate_interleaved")
        return out
    y = ref.rotate_interleaved(x, step.positions, inv_freq).to(out_dtype)
    if out is not None:
        out.copy_(y)
        return out
    return y


def clamped_glu_fused(gate_up, limit: float, alpha: float = 1.702):
    """(rows, 2I) [gate | up] -> g*sigmoid(alpha*g)*(u+1) with g = min(gate,
    limit), u = clamp(up, -limit, limit)."""
    I = gate_up.shape[-1] // 2
    if gate_up.is_cuda:
        lib = _load()
        gu = gate_up.contiguous()
        out = torch.empty(gu.shape[:-1] + (I,), dtype=gu.dtype, device=gu.device)
        _check(lib.nx_clamped_glu(_p(gu), _p(out), _is_bf16(gu),
                                  ctypes.c_long(gu.numel() // (2 * I)), I,
                                  ctypes.c_float(limit), ctypes.c_float(alpha), _stream()),
               "clamped_glu_fused")
        return out
    g, u = gate_up.chunk(2, dim=-1)
    return ref.clamped_glu(g, u, limit, alpha).to(gate_up.dtype)


def scaled_embedding(h, scale: float):
    """Embedding rows -> fp32 residual stream, times a constant."""
    return h.float().mul_(scale) if h.dtype != torch.float32 else h * scale


def head_norm_rotate(x, step: StepLayout, norm_weight, eps: float, inv_freq,
                     mscale: float = 1.0, out_dtype=None):
    """Per-head RMS norm (weight shared by the heads, None = none) and
    half-split rotary positions (channel i pairs with i + len(inv_freq), cos
    and sin times ``mscale``; None = no rotation) in one pass, statistics and
    angles in fp32. x (B,S,N,C), possibly a strided view of a fused
    projection; returns a dense (B,S,N*C) tensor."""
    out_dtype = out_dtype or x.dtype
    B, S, N, C = x.shape
    if x.is_cuda:
        lib = _load()
        out = torch.empty(B, S, N * C, dtype=out_dtype, device=x.device)
        assert x.stride(3) == 1
        half = 0 if inv_freq is None else inv_freq.numel()
        assert 2 * half <= C
        _check(lib.nx_head_norm_rope(
            _p(x), ctypes.c_long(_token_stride(x)), ctypes.c_long(x.stride(2)), _is_bf16(x),
            _p(out), _is_bf16(out), _p(step.positions),
            _p(None if norm_weight is None else _f32(norm_weight)), ctypes.c_float(eps),
            _p(None if half == 0 else _f32(inv_freq)), half, ctypes.c_float(mscale),
            ctypes.c_long(B * S), N, C, _stream()), "head_norm_rotate")
        return out
    return ref.head_norm_rotate(x, step.positions, norm_weight, eps, inv_freq,
                                mscale).reshape(B, S, N * C).to(out_dtype)


def decay_scan(q, k, v, state, step: StepLayout, dim: int, vdim: int, dt=None,
               dt_bias=None, a_log=None, head_decay=None, k_scale: float = 1.0, skip=None):
    """Scalar-decay linear recurrence with matrix state (see ref.decay_scan):
    selective state spaces (``dt``/``dt_bias``/``a_log``) or fixed per-head
    decays (``head_decay``). q, k (B,S,G*dim), v (B,S,H*vdim) may be column
    slices of wider tensors; ``state`` (slots, H, vdim, dim) fp32 is read
    (unless the row starts at position 0) and advanced. Returns fp32."""
    assert (dt is None) != (head_decay is None)
    if v.is_cuda:
        lib = _load()
        B, S = v.shape[0], v.shape[1]
        H = v.shape[-1] // vdim
        G = q.shape[-1] // dim
        assert q.dtype == k.dtype == v.dtype and state.dtype == torch.float32
        assert state.is_contiguous() and tuple(state.shape[1:]) == (H, vdim, dim)
        assert H % G == 0 and q.shape[-1] == G * dim and k.shape[-1] == G * dim
        out = torch.empty(B, S, H * vdim, dtype=torch.float32, device=v.device)
        # a long row with few (row, head, channel block) workgroups is cut into
        # segments that scan side by side (two passes joined by a short serial
        # link over the segments' end states)
        groups = B * H * ((vdim + 15) // 16)
        nseg, seglen, ws, wdec = 1, S, None, None
        if S >= 256 and groups < 1024:
            nseg = 1
            while nseg * 2 <= min(S // 64, max(1, 2048 // groups)):
                nseg *= 2
            if nseg > 1:
                seglen = ((S + nseg - 1) // nseg + 15) // 16 * 16
                ws = torch.empty(B * nseg * H * vdim * dim, dtype=torch.float32, device=v.device)
                wdec = torch.empty(B * nseg * H, dtype=torch.float32, device=v.device)
        _check(lib.nx_decay_scan(
            _p(q), ctypes.c_long(_rows_view(q)), _p(k), ctypes.c_long(_rows_view(k)),
            _p(v), ctypes.c_long(_rows_view(v)), _is_bf16(v),
            _p(dt), ctypes.c_long(0 if dt is None else _rows_view(dt)),
            0 if dt is None else _is_bf16(dt),
            _p(None if dt_bias is None else _f32(dt_bias)),
            _p(None if a_log is None else _f32(a_log)),
            _p(None if head_decay is None else _f32(head_decay)),
            ctypes.c_float(k_scale), _p(None if skip is None else _f32(skip)),
            _p(state), _p(step.positions), _p(step.seq_ids), _p(step.nvalid), _p(out),
            B, S, H, G, dim, vdim, _p(ws), _p(wdec), nseg, seglen, _stream()), "decay_scan")
        return out
    return ref.decay_scan(q, k, v, state, step.positions, step.seq_ids, dim, vdim,
                          dt=dt, dt_bias=dt_bias, a_log=a_log, head_decay=head_decay,
                          k_scale=k_scale, skip=skip)


def group_gated_norm(y, gate, weight, eps: float, groups: int, gate_first: bool,
                     out_dtype=torch.float32):
    """RMS norm of fp32 rows in ``groups`` equal parts with a silu gate before
    or after it and an optional weight (see ref.group_gated_norm). ``gate``
    may be a column slice of a wider tensor."""
    if y.is_cuda:
        lib = _load()
        C = y.shape[-1]
        assert y.dtype == torch.float32 and y.is_contiguous() and C % groups == 0
        out = torch.empty(y.shape, dtype=out_dtype, device=y.device)
        _check(lib.nx_group_gated_norm(
            _p(y), _p(gate), ctypes.c_long(_rows_view(gate)), _is_bf16(gate),
            _p(None if weight is None else _f32(weight)), ctypes.c_float(eps), groups,
            int(gate_first), _p(out), _is_bf16(out), ctypes.c_long(y.numel() // C), C,
            _stream()), "group_gated_norm")
        return out
    return ref.group_gated_norm(y, gate, weight, eps, groups, gate_first, out_dtype)


def group_limited_router(logits, num_experts: int, top_k: int, n_groups: int = 1,
                         keep_groups: int = 1, scale: float = 1.0, normalize: bool = False,
                         correction=None):
    """Group-limited top-k routing on fp32 logits (T, E + extra) (see
    ref.group_limited_router; ``correction`` (E,) shifts the scores for the
    choice only): returns (dense (T, E + extra) weights with
    sigmoid gates in the extra columns, idx (T, top_k) int32, weights)."""
    if logits.is_cuda:
        lib = _load()
        T, C = logits.shape
        E = num_experts
        assert logits.dtype == torch.float32 and logits.stride(1) == 1
        assert E % max(n_groups, 1) == 0 and top_k <= E
        dense = torch.empty(T, C, dtype=torch.float32, device=logits.device)
        idx = torch.empty(T, top_k, dtype=torch.int32, device=logits.device)
        wts = torch.empty(T, top_k, dtype=torch.float32, device=logits.device)
        _check(lib.nx_group_router(
            _p(logits), ctypes.c_long(logits.stride(0)), E, C - E, top_k, max(n_groups, 1),
            max(min(keep_groups, n_groups), 1), ctypes.c_float(scale), int(normalize),
            _p(None if correction is None else _f32(correction)),
            _p(dense), _p(idx), _p(wts), ctypes.c_long(T), _stream()), "group_limited_router")
        return dense, idx, wts
    return ref.group_limited_router(logits, num_experts, top_k, max(n_groups, 1),
                                    max(min(keep_groups, n_groups), 1), scale, normalize,
                                    correction)


FUSED_ROUTER_MAX_TOKENS = 512


def route_tokens(x, weight, num_experts: int, top_k: int, n_groups: int = 1,
                 keep_groups: int = 1, scale: float = 1.0, normalize: bool = False,
                 correction=None):
    """Router product and selection: fp32 logits ``x.float() @ weight.T`` (x
    (T, hidden) in any dtype, weight (E + extra, hidden) fp32), then
    :func:`group_limited_router`. Steps of few tokens do both in one launch;
    larger ones take the library product first."""
    T = x.shape[0]
    if x.is_cuda and 0 < T <= FUSED_ROUTER_MAX_TOKENS and x.stride(-1) == 1:
        lib = _load()
        E, C = num_experts, weight.shape[0]
        assert weight.dtype == torch.float32 and weight.is_contiguous()
        assert weight.shape[1] == x.shape[1] and E % max(n_groups, 1) == 0 and top_k <= E
        dense = torch.empty(T, C, dtype=torch.float32, device=x.device)
        idx = torch.empty(T, top_k, dtype=torch.int32, device=x.device)
        wts = torch.empty(T, top_k, dtype=torch.float32, device=x.device)
        _check(lib.nx_router_fused(
            _p(x), ctypes.c_long(x.stride(0)), _is_bf16(x), _p(weight), weight.shape[1], E, C - E,
            top_k, max(n_groups, 1), max(min(keep_groups, n_groups), 1), ctypes.c_float(scale),
            int(normalize), _p(None if correction is None else _f32(correction)),
            _p(dense), _p(idx), _p(wts), ctypes.c_long(T), _stream()), "route_tokens")
        return dense, idx, wts
    logits = torch.nn.functional.linear(x.float(), weight)
    return group_limited_router(logits, num_experts, top_k, n_groups, keep_groups, scale,
                                normalize, correction=correction)


def latent_row_write(x, norm_weight, eps: float, inv_freq, step: StepLayout, k_cache,
                     slot_mapping, kv_rank: int, row=None):
    """Cache row of a latent layer in one pass: x (B,S,kv_rank + rot) (a column
    slice is fine) -> [rms_norm(x[..., :kv_rank]) * w | interleaved-pair rotary
    of the rest] scattered into the paged ``k_cache`` (blocks, block, 1,
    kv_rank + rot) at ``slot_mapping``; ``row`` (B,S,kv_rank + rot, dense)
    also receives it when given."""
    B, S, CR = x.shape
    C, R = kv_rank, CR - kv_rank
    if x.is_cuda:
        lib = _load()
        assert k_cache.is_contiguous() and k_cache.shape[2] * k_cache.shape[3] == CR
        assert k_cache.dtype == x.dtype and x.stride(2) == 1
        assert row is None or (row.is_contiguous() and row.dtype == x.dtype and row.shape == x.shape)
        _check(lib.nx_latent_row(
            _p(x), ctypes.c_long(_token_stride(x)), _is_bf16(x), _p(_f32(norm_weight)),
            ctypes.c_float(eps), _p(_f32(inv_freq)), inv_freq.numel(), _p(step.positions),
            _p(step.i32(slot_mapping)), _p(k_cache),
            ctypes.c_long(k_cache.shape[0] * k_cache.shape[1]), _p(row),
            ctypes.c_long(0 if row is None else CR), ctypes.c_long(B * S), C, R, _stream()),
            "latent_row_write")
        return row
    r = torch.empty(B, S, CR, dtype=x.dtype, device=x.device)
    r[..., :C] = ref.rms_norm_rows(x[..., :C], norm_weight, eps, False, x.dtype)
    r[..., C:] = ref.rotate_interleaved(x[..., C:].unsqueeze(2), step.positions,
                                        inv_freq).squeeze(2).to(x.dtype)
    ref.paged_kv_write(k_cache, None, r.view(B * S, 1, CR), None, slot_mapping)
    if row is not None:
        row.copy_(r)
    return row


def relu2_scale(hid, gates, expert_ff: int, num_experts: int, out_dtype=None):
    """relu(x)^2 of (T, E*ff + rest) pre-activations times the token's gate of
    the column's expert; the remaining columns take gate column E (see
    ref.relu2_scale). ``gates`` None: plain relu(x)^2."""
    out_dtype = out_dtype or hid.dtype
    if hid.is_cuda:
        lib = _load()
        T, C = hid.shape
        assert hid.is_contiguous() and out_dtype == hid.dtype
        out = torch.empty(T, C, dtype=out_dtype, device=hid.device)
        if gates is None:
            _check(lib.nx_relu2_scale(_p(hid), _is_bf16(hid), _p(None), 0, max(C, 1), 1,
                                      _p(out), ctypes.c_long(T), C, _stream()), "relu2_scale")
            return out
        assert gates.dtype == torch.float32 and gates.is_contiguous()
        assert C == num_experts * expert_ff or gates.shape[1] == num_experts + 1
        _check(lib.nx_relu2_scale(_p(hid), _is_bf16(hid), _p(gates), gates.shape[1], expert_ff,
                                  num_experts, _p(out), ctypes.c_long(T), C, _stream()),
               "relu2_scale")
        return out
    return ref.relu2_scale(hid, gates, expert_ff, num_experts, out_dtype)


def clamped_glu_scale(hid, gates, expert_ff: int, num_experts: int, limit: float,
                      shared_limit: float = 0.0, alpha: float = 1.702, out_dtype=None):
    """Clamped gated units of stacked experts (see ref.clamped_glu_scale):
    hid (T, 2*C) = [gate | up] of C = E*ff + shared columns -> (T, C), an
    expert's columns times the token's routing weight ``gates[t, e]`` (fp32,
    (T, >= E), row-strided), the shared columns with their own clamp."""
    out_dtype = out_dtype or hid.dtype
    if hid.is_cuda:
        lib = _load()
        T, C2 = hid.shape
        C = C2 // 2
        assert hid.is_contiguous() and out_dtype == hid.dtype and C2 == 2 * C
        assert num_experts * expert_ff <= C
        if num_experts:
            assert gates.dtype == torch.float32 and gates.stride(1) == 1
            assert gates.shape[0] == T and gates.shape[1] >= num_experts
        out = torch.empty(T, C, dtype=out_dtype, device=hid.device)
        _check(lib.nx_clamped_glu_scale(
            _p(hid), _is_bf16(hid), _p(gates if num_experts else None),
            ctypes.c_long(gates.stride(0) if num_experts else 0), expert_ff, num_experts,
            ctypes.c_float(limit), ctypes.c_float(shared_limit), ctypes.c_float(alpha),
            _p(out), ctypes.c_long(T), C, _stream()), "clamped_glu_scale")
        return out
    return ref.clamped_glu_scale(hid, gates, expert_ff, num_experts, limit, shared_limit,
                                 alpha, out_dtype)


def sigmoid_gate_(y, gate):
    """In place: y *= sigmoid(gate). y (..., C) contiguous; ``gate`` of the
    same shape may be a column slice of a wider tensor."""
    if y.is_cuda:
        lib = _load()
        C = y.shape[-1]
        assert y.is_contiguous() and gate.shape == y.shape and gate.dtype == y.dtype
        _check(lib.nx_sigmoid_gate(_p(y), _p(gate), ctypes.c_long(_rows_view(gate)), _is_bf16(y),
                                   ctypes.c_long(y.numel() // C), C, _stream()), "sigmoid_gate")
        return y
    return y.copy_(y.float() * torch.sigmoid(gate.float()))


def scaled_residual(x, terms, eps: float = 0.0):
    """In place on the fp32 stream: x += sum_i f_i(y_i) * w_i for up to three
    terms (y (..., C) in one dtype, w (C,) fp32, normed): f_i is an RMS norm
    over the row (with ``eps``) when ``normed`` else the identity."""
    assert 1 <= len(terms) <= 3
    if x.is_cuda:
        lib = _load()
        C = x.shape[-1]
        assert x.dtype == torch.float32 and x.is_contiguous()
        args = []
        keep = []
        for i in range(3):
            if i < len(terms):
                y, w, normed = terms[i]
                y = y.contiguous()
                assert y.dtype == terms[0][0].dtype and y.numel() == x.numel()
                wf = _f32(w)
                keep += [y, wf]
                args += [_p(y), _p(wf), int(bool(normed))]
            else:
                args += [_p(None), _p(None), 0]
        _check(lib.nx_scaled_residual(_p(x), *args, _is_bf16(terms[0][0]), ctypes.c_float(eps),
                                      ctypes.c_long(x.numel() // C), C, _stream()),
               "scaled_residual")
        return x
    return ref.scaled_residual(x, [(y, w, eps if normed else None) for y, w, normed in terms])


def embed_positions(h, pos_table, step: StepLayout):
    """Token embedding rows (B,S,W) plus a learned position row per token ->
    fp32 residual stream; pad tokens (position -1) take row 0."""
    if h.is_cuda:
        lib = _load()
        h = h.contiguous()
        assert pos_table.dtype == h.dtype and pos_table.is_contiguous()
        W = h.shape[-1]
        out = torch.empty(h.shape, dtype=torch.float32, device=h.device)
        _check(lib.nx_embed_pos(_p(h), _p(pos_table), _is_bf16(h), _p(step.positions), _p(out),
                                ctypes.c_long(h.numel() // W), W, pos_table.shape[0], _stream()),
               "embed_positions")
        return out
    p = step.positions.long().clamp(min=0, max=pos_table.shape[0] - 1)
    return h.float() + pos_table[p].float()

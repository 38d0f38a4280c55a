"""Tensor-level wrappers over the C ABI: they validate, allocate outputs with torch and pass raw
device pointers + the current HIP stream.  No arithmetic happens here and nothing falls back to
torch ops: a CPU tensor or a missing library is an error.
"""
from __future__ import annotations

import ctypes
from typing import Optional, Tuple

import torch

from . import _lib
from ._lib import MAX_KV_CHUNKS, PICO_BF16, PICO_F32, AttnDesc, KvChunks, RopeTables, check

_DT = {torch.bfloat16: PICO_BF16, torch.float32: PICO_F32}


def _dt(t: torch.Tensor, what: str) -> int:
    if t.dtype not in _DT:
        raise RuntimeError(f"{what}: dtype {t.dtype} not supported by the HIP kernels (bf16 / fp32 only)")
    return _DT[t.dtype]


def _dev(*tensors: Optional[torch.Tensor]) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("picotron_amd kernels run on the GPU only: got a CPU tensor (there is no CPU fallback)")


def _ptr(t: Optional[torch.Tensor]):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


# ------------------------------------------------------------------------------- RMSNorm
def rmsnorm_fwd(x: torch.Tensor, weight: torch.Tensor, eps: float, cast_then_scale: bool,
                residual: Optional[torch.Tensor] = None, want_residual_out: bool = False,
                want_rstd: bool = True):
    """Returns (y, rstd or None, residual_out or None); x is [..., hidden]."""
    _dev(x, weight, residual)
    hidden = x.size(-1)
    xc = x.contiguous()
    w = weight.to(x.dtype).contiguous() if weight.dtype != x.dtype else weight.contiguous()
    rows = xc.numel() // hidden if hidden else 0
    y = torch.empty_like(xc)
    rstd = torch.empty(rows, dtype=torch.float32, device=x.device) if want_rstd else None
    res = residual.contiguous() if residual is not None else None
    if res is not None and (res.dtype != x.dtype or res.shape != x.shape):
        raise RuntimeError("rmsnorm_fwd: residual must match x in dtype and shape")
    res_out = torch.empty_like(xc) if (res is not None and want_residual_out) else None
    check(_lib.lib().pico_rmsnorm_fwd(_ptr(xc), _ptr(w), _ptr(y), _ptr(rstd), _ptr(res), _ptr(res_out), rows, hidden,
                                      float(eps), int(cast_then_scale), _dt(x, "rmsnorm_fwd"), _stream()))
    return y, rstd, res_out


def rmsnorm_bwd(dy: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, rstd: torch.Tensor,
                dresidual: Optional[torch.Tensor] = None, dw_dtype=torch.float32):
    """Returns (dx in x.dtype, dweight [hidden] in dw_dtype).  `dresidual` (x's shape and dtype), when given, is added
    to dx inside the kernel: the gradient that reached the residual stream directly."""
    _dev(dy, x, weight, rstd, dresidual)
    hidden = x.size(-1)
    xc, dyc = x.contiguous(), dy.contiguous()
    if dyc.dtype != xc.dtype:
        dyc = dyc.to(xc.dtype)
    if dresidual is not None:
        if dresidual.shape != x.shape:
            raise RuntimeError("rmsnorm_bwd: dresidual must have x's shape")
        dresidual = dresidual.contiguous()
        if dresidual.dtype != xc.dtype:
            dresidual = dresidual.to(xc.dtype)
    w = weight.to(x.dtype).contiguous() if weight.dtype != x.dtype else weight.contiguous()
    rows = xc.numel() // hidden if hidden else 0
    dx = torch.empty_like(xc)
    dw = torch.empty(hidden, dtype=dw_dtype, device=x.device)
    ws_bytes = _lib.lib().pico_rmsnorm_bwd_workspace_bytes(rows, hidden)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=x.device)
    check(_lib.lib().pico_rmsnorm_bwd(_ptr(dyc), _ptr(xc), _ptr(w), _ptr(rstd), _ptr(dresidual), _ptr(dx), _ptr(dw),
                                      _dt(dw, "rmsnorm_bwd dweight"), _ptr(ws), ws_bytes, rows, hidden,
                                      _dt(x, "rmsnorm_bwd"), _stream()))
    return dx, dw


# ------------------------------------------------------------------------------- RoPE
def rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, pos_offset: int = 0, inverse: bool = False,
         out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Rotates x [B,H,S,D] (any b/h/s strides, unit D stride) with table rows pos_offset + s."""
    _dev(x, cos, sin, out)
    if x.dim() != 4:
        raise RuntimeError("rope: x must be [B, H, S, D]")
    if x.stride(-1) != 1:
        x = x.contiguous()
    if cos.dtype != sin.dtype or cos.stride(-1) != 1 or sin.stride(-1) != 1 or cos.stride(0) != sin.stride(0):
        raise RuntimeError("rope: cos and sin must share dtype and row pitch, with contiguous rows")
    B, H, S, D = x.shape
    if cos.size(0) < pos_offset + S:
        raise RuntimeError(f"rope: tables have {cos.size(0)} rows, need {pos_offset + S}")
    if out is None:
        # keep the memory order of x so that a transposed view stays a free view downstream
        out = torch.empty_strided(x.shape, x.stride(), dtype=x.dtype, device=x.device) if _dense(x) else torch.empty_like(x)
    check(_lib.lib().pico_rope(_ptr(x), _ptr(out), _ptr(cos), _ptr(sin), B, H, S, D,
                               x.stride(0), x.stride(1), x.stride(2), out.stride(0), out.stride(1), out.stride(2),
                               cos.stride(0), int(pos_offset), int(inverse), _dt(cos, "rope tables"), _dt(x, "rope"),
                               _stream()))
    return out


def _dense(t: torch.Tensor) -> bool:
    """True if t's strides are a permutation of a contiguous layout (no gaps, no overlap)."""
    dims = sorted(range(t.dim()), key=lambda i: t.stride(i), reverse=True)
    expect = 1
    for i in reversed(dims):
        if t.size(i) != 1 and t.stride(i) != expect:
            return False
        expect *= t.size(i)
    return True


# ------------------------------------------------------------------------------- SwiGLU
def _as_2d(t: torch.Tensor) -> torch.Tensor:
    """[..., C] -> [rows, C] without a copy when the leading dims collapse to one row pitch (a column slice of a
    contiguous buffer does); a copy otherwise."""
    if t.stride(-1) != 1:
        t = t.contiguous()
    if t.dim() == 2:
        return t
    try:
        return t.view(-1, t.size(-1))
    except RuntimeError:
        pass
    # leading dims with a common pitch: stride[i] == stride[i+1] * size[i+1]
    if all(t.stride(i) == t.stride(i + 1) * t.size(i + 1) for i in range(t.dim() - 2)):
        rows = t.numel() // t.size(-1)
        return t.as_strided((rows, t.size(-1)), (t.stride(-2), 1))
    return t.contiguous().view(-1, t.size(-1))


def swiglu_fwd(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    _dev(gate, up)
    if gate.shape != up.shape or gate.dtype != up.dtype:
        raise RuntimeError("swiglu_fwd: gate and up must match")
    g2, u2 = _as_2d(gate), _as_2d(up)
    y = torch.empty(gate.shape, dtype=gate.dtype, device=gate.device)
    y2 = y.view(-1, y.size(-1))
    check(_lib.lib().pico_swiglu_fwd(_ptr(g2), _ptr(u2), _ptr(y2), g2.size(0), g2.size(1), g2.stride(0), u2.stride(0),
                                     y2.stride(0), _dt(gate, "swiglu_fwd"), _stream()))
    return y


def swiglu_bwd(dy: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, out=None):
    """(dgate, dup); `out` = (dgate, dup) buffers to write into (e.g. the two halves of one fused gradient)."""
    _dev(dy, gate, up)
    g2, u2, d2 = _as_2d(gate), _as_2d(up), _as_2d(dy.to(gate.dtype))
    if out is None:
        dg = torch.empty(gate.shape, dtype=gate.dtype, device=gate.device)
        du = torch.empty(gate.shape, dtype=gate.dtype, device=gate.device)
    else:
        dg, du = out
        if dg.shape != gate.shape or du.shape != gate.shape or dg.dtype != gate.dtype or du.dtype != gate.dtype:
            raise RuntimeError("swiglu_bwd: out buffers must match gate in shape and dtype")
    dg2, du2 = _as_2d(dg), _as_2d(du)
    if dg2.data_ptr() != dg.data_ptr() or du2.data_ptr() != du.data_ptr():
        raise RuntimeError("swiglu_bwd: out buffers need a unit last stride and one row pitch")
    check(_lib.lib().pico_swiglu_bwd(_ptr(d2), _ptr(g2), _ptr(u2), _ptr(dg2), _ptr(du2), g2.size(0), g2.size(1),
                                     d2.stride(0), g2.stride(0), u2.stride(0), dg2.stride(0), du2.stride(0),
                                     _dt(gate, "swiglu_bwd"), _stream()))
    return dg, du


# ------------------------------------------------------------------------------- lse merge
def lse_merge_(out: torch.Tensor, lse: torch.Tensor, block_out: torch.Tensor, block_lse: torch.Tensor) -> None:
    """In place: (out fp32 [..., D], lse fp32 [...]) <- merge with (block_out, block_lse)."""
    _dev(out, lse, block_out, block_lse)
    if out.dtype != torch.float32 or lse.dtype != torch.float32 or block_lse.dtype != torch.float32:
        raise RuntimeError("lse_merge_: out, lse and block_lse must be fp32")
    if not (out.is_contiguous() and lse.is_contiguous()):
        raise RuntimeError("lse_merge_: out and lse must be contiguous (they are updated in place)")
    D = out.size(-1)
    rows = out.numel() // D
    bo, bl = block_out.contiguous(), block_lse.contiguous()
    check(_lib.lib().pico_lse_merge(_ptr(out), _ptr(lse), _ptr(bo), _ptr(bl), rows, D, _dt(bo, "lse_merge_"), _stream()))


# ------------------------------------------------------------------------------- attention
def _desc(q, k, v, o, sm_scale, causal, q_offset) -> AttnDesc:
    B, Hq, Sq, D = q.shape
    Hkv, Sk = k.size(1), k.size(2)
    d = AttnDesc()
    d.B, d.Hq, d.Hkv, d.Sq, d.Sk, d.D = B, Hq, Hkv, Sq, Sk, D
    d.causal, d.q_offset, d.sm_scale = int(bool(causal)), int(q_offset), float(sm_scale)
    for name, t in (("q_stride", q), ("k_stride", k), ("v_stride", v), ("o_stride", o)):
        arr = getattr(d, name)
        arr[0], arr[1], arr[2] = t.stride(0), t.stride(1), t.stride(2)
    return d


def _attn_in(t: torch.Tensor, what: str) -> torch.Tensor:
    if t.dtype != torch.bfloat16:
        raise RuntimeError(f"attention: {what} must be bf16 (got {t.dtype}); the MFMA kernels are bf16 only")
    if t.dim() != 4:
        raise RuntimeError(f"attention: {what} must be [B, H, S, D]")
    if t.stride(-1) != 1 or any(s % 8 for s in t.stride()[:3]):
        t = t.contiguous()
    return t


def empty_bshd(B: int, H: int, S: int, D: int, dtype, device) -> torch.Tensor:
    """A [B,H,S,D]-shaped view of a fresh [B,S,H,D] buffer: `.transpose(1,2).reshape(B,S,H*D)` on it is free."""
    return torch.empty(B, S, H, D, dtype=dtype, device=device).transpose(1, 2)


def attn_fwd(q, k, v, sm_scale: float, causal: bool, q_offset: int = 0, out: Optional[torch.Tensor] = None,
             lse: Optional[torch.Tensor] = None, merge: bool = False, out_dtype=torch.bfloat16,
             bshd_out: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """softmax(q k^T * scale + mask) v for q [B,Hq,Sq,D], k/v [B,Hkv,Sk,D]; returns (out, lse fp32 [B,Hq,Sq]).

    merge=True continues the online softmax from the running fp32 (out, lse) passed in and updates them in place.
    """
    _dev(q, k, v, out, lse)
    q, k, v = _attn_in(q, "q"), _attn_in(k, "k"), _attn_in(v, "v")
    B, Hq, Sq, D = q.shape
    if k.shape != v.shape or k.size(0) != B or k.size(3) != D:
        raise RuntimeError(f"attention: shape mismatch q{tuple(q.shape)} k{tuple(k.shape)} v{tuple(v.shape)}")
    if merge:
        if out is None or lse is None or out.dtype != torch.float32:
            raise RuntimeError("attn_fwd(merge=True) needs the running fp32 out and lse")
    if out is None:
        out = empty_bshd(B, Hq, Sq, D, out_dtype, q.device) if bshd_out else torch.empty(B, Hq, Sq, D, dtype=out_dtype, device=q.device)
    if lse is None:
        lse = torch.empty(B, Hq, Sq, dtype=torch.float32, device=q.device)
    if not lse.is_contiguous() or lse.dtype != torch.float32 or out.stride(-1) != 1:
        raise RuntimeError("attn_fwd: lse must be contiguous fp32 and out must have a unit D stride")
    d = _desc(q, k, v, out, sm_scale, causal, q_offset)
    check(_lib.lib().pico_attn_fwd(ctypes.byref(d), _ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lse), _dt(out, "attn_fwd out"),
                                   int(merge), _stream()))
    return out, lse


def _rope_tables(cos: torch.Tensor, sin: torch.Tensor) -> RopeTables:
    _dev(cos, sin)
    if cos.dtype != sin.dtype or cos.dim() != 2 or cos.shape != sin.shape or cos.stride(-1) != 1 or sin.stride(-1) != 1 \
            or cos.stride(0) != sin.stride(0):
        raise RuntimeError("rope tables: cos and sin must be [positions, columns] of one dtype and row pitch, with contiguous rows")
    t = RopeTables()
    t.cos, t.sin, t.pitch, t.dtype, t.rows = cos.data_ptr(), sin.data_ptr(), cos.stride(0), _dt(cos, "rope tables"), cos.size(0)
    return t


def attn_fwd_rope(q, k_rot, v, cos, sin, sm_scale: float, causal: bool, q_offset: int = 0, q_pos_offset: int = 0,
                  want_q_rot: bool = True, out_dtype=torch.bfloat16, bshd_out: bool = True, out=None, lse=None,
                  merge: bool = False, q_rot=None):
    """RoPE on q inside the attention forward (k_rot must be rotated already): returns (out, lse, q_rot or None); q_rot is
    the rotated q, laid out like q, for attn_bwd_rope.  merge=True continues from the running fp32 (out, lse) given, as
    attn_fwd does: one step of a ring whose queries sit at positions q_pos_offset .."""
    _dev(q, k_rot, v, out, lse, q_rot)
    q, k_rot, v = _attn_in(q, "q"), _attn_in(k_rot, "k"), _attn_in(v, "v")
    B, Hq, Sq, D = q.shape
    if k_rot.shape != v.shape or k_rot.size(0) != B or k_rot.size(3) != D:
        raise RuntimeError(f"attention: shape mismatch q{tuple(q.shape)} k{tuple(k_rot.shape)} v{tuple(v.shape)}")
    if merge and (out is None or lse is None or out.dtype != torch.float32):
        raise RuntimeError("attn_fwd_rope(merge=True) needs the running fp32 out and lse")
    if out is None:
        out = empty_bshd(B, Hq, Sq, D, out_dtype, q.device) if bshd_out else torch.empty(B, Hq, Sq, D, dtype=out_dtype, device=q.device)
    if lse is None:
        lse = torch.empty(B, Hq, Sq, dtype=torch.float32, device=q.device)
    if not lse.is_contiguous() or lse.dtype != torch.float32 or out.stride(-1) != 1:
        raise RuntimeError("attn_fwd_rope: lse must be contiguous fp32 and out must have a unit D stride")
    qrs = None
    if want_q_rot and q_rot is None:
        q_rot = empty_bshd(B, Hq, Sq, D, q.dtype, q.device)
    if q_rot is not None:
        qrs = (ctypes.c_int64 * 3)(*q_rot.stride()[:3])
    tables = _rope_tables(cos, sin)
    d = _desc(q, k_rot, v, out, sm_scale, causal, q_offset)
    check(_lib.lib().pico_attn_fwd_rope(ctypes.byref(d), _ptr(q), _ptr(k_rot), _ptr(v), _ptr(out), _ptr(lse), _dt(out, "attn out"),
                                        int(merge), ctypes.byref(tables), int(q_pos_offset), _ptr(q_rot), qrs, _stream()))
    return out, lse, q_rot


def attn_bwd_rope(dout, q_rot, k_rot, v, out, lse, cos, sin, sm_scale: float, causal: bool, dq, dk, dv, q_offset: int = 0,
                  q_pos_offset: int = 0, k_pos_offset: int = 0, dq_accumulate: bool = False, dkv_accumulate: bool = False):
    """Backward of "rotate q and k, attend": writes (or, with the accumulate flags, adds to the fp32) dq / dk -- gradients
    of the UN-rotated q and k: RoPE's backward runs in the kernels' epilogues -- and dv in the given buffers (any strides
    with a unit D stride)."""
    _dev(dout, q_rot, k_rot, v, out, lse, dq, dk, dv)
    q_rot, k_rot, v, dout = _attn_in(q_rot, "q"), _attn_in(k_rot, "k"), _attn_in(v, "v"), _attn_in(dout, "dout")
    if out.stride() != dout.stride():
        out = _like_strided(out, dout)
    if out.dtype != torch.bfloat16:
        raise RuntimeError("attn_bwd_rope: out must be the bf16 forward output")
    B, Hq, Sq, D = q_rot.shape
    if dk.dtype != dv.dtype or dk.stride() != dv.stride() or dk.stride(-1) != 1 or dq.stride(-1) != 1:
        raise RuntimeError("attn_bwd_rope: dk and dv must share dtype and strides; dq, dk, dv need a unit D stride")
    delta = torch.empty(B, Hq, Sq, dtype=torch.float32, device=q_rot.device)
    tables = _rope_tables(cos, sin)
    d = _desc(q_rot, k_rot, v, dout, sm_scale, causal, q_offset)
    dqs = (ctypes.c_int64 * 3)(*dq.stride()[:3])
    dks = (ctypes.c_int64 * 3)(*dk.stride()[:3])
    check(_lib.lib().pico_attn_bwd_rope(ctypes.byref(d), _ptr(q_rot), _ptr(k_rot), _ptr(v), _ptr(dout), _ptr(out),
                                        _ptr(lse.contiguous()), _ptr(delta), _ptr(dq), dqs, _dt(dq, "dq"), int(dq_accumulate),
                                        _ptr(dk), _ptr(dv), dks, _dt(dk, "dk/dv"), int(dkv_accumulate), ctypes.byref(tables),
                                        int(q_pos_offset), int(k_pos_offset), _stream()))
    return dq, dk, dv


# ---- all ring steps of one rank in one launch: K / V as a list of equally shaped chunk tensors
FINAL_TOTAL_DTYPES = (torch.bfloat16,)   # dtypes attn_bwd_chunks can write a chunk's rounded totals in (dk_finals / dv_finals)


def chunks_fit_one_launch(ks, vs) -> bool:
    """True if the chunk tensors can go to the chunk-list entry points as they are: at most 16 bf16 chunks of one shape
    and one stride triple (k's may differ from v's), unit D stride, strides that are multiples of 8, and -- with several
    chunks -- a chunk length that is a multiple of 128 (no staged key tile straddles two chunks)."""
    if not ks or len(ks) != len(vs) or len(ks) > MAX_KV_CHUNKS:
        return False
    k0, v0 = ks[0], vs[0]
    if k0.dim() != 4 or (len(ks) > 1 and k0.size(2) % 128 != 0):
        return False
    shape, ksd, vsd, bf16 = k0.shape, k0.stride(), v0.stride(), torch.bfloat16
    if (v0.dim() != 4 or ksd[3] != 1 or vsd[3] != 1 or ksd[0] % 8 or ksd[1] % 8 or ksd[2] % 8
            or vsd[0] % 8 or vsd[1] % 8 or vsd[2] % 8):
        return False
    for k, v in zip(ks, vs):      # (this runs once per attention call of every layer: kept flat)
        if (k.dtype != bf16 or v.dtype != bf16 or k.shape != shape or v.shape != shape or k.stride() != ksd
                or v.stride() != vsd or k.data_ptr() % 16 or v.data_ptr() % 16 or not k.is_cuda or not v.is_cuda):
            return False
    return True


def _kv_chunks(ks, vs, dks=None, dvs=None, accumulate=None, dk_finals=None, dv_finals=None) -> KvChunks:
    c = KvChunks()
    c.count, c.chunk_len = len(ks), ks[0].size(2)
    mask = 0
    for i, (k, v) in enumerate(zip(ks, vs)):
        c.k[i], c.v[i] = k.data_ptr(), v.data_ptr()
        if dks is not None and dks[i] is not None:
            c.dk[i], c.dv[i] = dks[i].data_ptr(), dvs[i].data_ptr()
            if accumulate is not None and accumulate[i]:
                mask |= 1 << i
        if dk_finals is not None and dk_finals[i] is not None:
            c.dk_final[i], c.dv_final[i] = dk_finals[i].data_ptr(), dv_finals[i].data_ptr()
            c.final_stride[0], c.final_stride[1], c.final_stride[2] = dk_finals[i].stride()[:3]
    c.accumulate_mask = mask
    return c


def _chunk_desc(q, ks, vs, o, sm_scale, causal, q_offset) -> AttnDesc:
    d = _desc(q, ks[0], vs[0], o, sm_scale, causal, q_offset)
    d.Sk = len(ks) * ks[0].size(2)
    return d


def attn_fwd_chunks(q, ks, vs, sm_scale: float, causal: bool, q_offset: int = 0, out=None, lse=None, merge: bool = False,
                    out_dtype=torch.bfloat16, bshd_out: bool = False, rope=None, q_pos_offset: int = 0,
                    want_q_rot: bool = False, checked: bool = False):
    """attn_fwd over K / V given as lists of chunk tensors (see chunks_fit_one_launch) that follow each other along the
    key axis: key j sits at position j of the concatenation, which is never materialised.  rope = (cos, sin): q is
    rotated inside the kernel (the chunks' k must be rotated already).  Returns (out, lse, q_rot or None)."""
    _dev(q, out, lse)
    if not checked and not chunks_fit_one_launch(ks, vs):     # checked: the caller has asked chunks_fit_one_launch already
        raise RuntimeError("attn_fwd_chunks: the chunks do not fit one launch (see chunks_fit_one_launch)")
    q = _attn_in(q, "q")
    B, Hq, Sq, D = q.shape
    if ks[0].size(0) != B or ks[0].size(3) != D:
        raise RuntimeError(f"attention: shape mismatch q{tuple(q.shape)} k{tuple(ks[0].shape)}")
    if merge and (out is None or lse is None or out.dtype != torch.float32):
        raise RuntimeError("attn_fwd_chunks(merge=True) needs the running fp32 out and lse")
    if out is None:
        out = empty_bshd(B, Hq, Sq, D, out_dtype, q.device) if bshd_out else torch.empty(B, Hq, Sq, D, dtype=out_dtype, device=q.device)
    if lse is None:
        lse = torch.empty(B, Hq, Sq, dtype=torch.float32, device=q.device)
    if not lse.is_contiguous() or lse.dtype != torch.float32 or out.stride(-1) != 1:
        raise RuntimeError("attn_fwd_chunks: lse must be contiguous fp32 and out must have a unit D stride")
    d = _chunk_desc(q, ks, vs, out, sm_scale, causal, q_offset)
    kv = _kv_chunks(ks, vs)
    tables = q_rot = qrs = None
    if rope is not None:
        tables = ctypes.byref(_rope_tables(*rope))
        if want_q_rot:
            q_rot = empty_bshd(B, Hq, Sq, D, q.dtype, q.device)
            qrs = (ctypes.c_int64 * 3)(*q_rot.stride()[:3])
    check(_lib.lib().pico_attn_fwd_chunks(ctypes.byref(d), _ptr(q), ctypes.byref(kv), _ptr(out), _ptr(lse), _dt(out, "attn out"),
                                          int(merge), tables, int(q_pos_offset), _ptr(q_rot), qrs, _stream()))
    return out, lse, q_rot


def attn_bwd_chunks(dout, q, ks, vs, lse, sm_scale: float, causal: bool, q_offset: int = 0, dq=None, dks=None, dvs=None,
                    dq_accumulate: bool = False, dkv_accumulate=None, out=None, delta=None, rope=None,
                    q_pos_offset: int = 0, k_pos_offset: int = 0, dk_finals=None, dv_finals=None, checked: bool = False):
    """attn_bwd over a chunk list.  dks / dvs: per chunk a gradient buffer (all of one dtype and stride triple) or None
    (not wanted); dkv_accumulate: per chunk, add to the fp32 buffer instead of writing it.  dq None: not wanted.  With
    `out` (forward output) delta is computed inside the call, otherwise `delta` must be given.  rope = (cos, sin): q and
    the chunks' k are rotated tensors, dq / dk leave un-rotated.  dk_finals / dv_finals: per chunk a bf16 buffer (all of
    one stride triple) or None; where given, this call holds the last block the chunk's gradient waits for, and the
    total -- the fp32 sums in dks / dvs (if the chunk's dkv_accumulate flag is set) plus this block -- is written there,
    rounded once; the fp32 buffers are only read.  Returns delta."""
    _dev(dout, q, lse, dq, out, delta)
    if not checked and not chunks_fit_one_launch(ks, vs):
        raise RuntimeError("attn_bwd_chunks: the chunks do not fit one launch (see chunks_fit_one_launch)")
    q, dout = _attn_in(q, "q"), _attn_in(dout, "dout")
    B, Hq, Sq, D = q.shape
    if out is not None and out.stride() != dout.stride():
        out = _like_strided(out, dout)
    if delta is None:
        if out is None:
            raise RuntimeError("attn_bwd_chunks: delta (or out, to compute it) is required")
        delta = torch.empty(B, Hq, Sq, dtype=torch.float32, device=q.device)
    if not (delta.is_contiguous() and delta.dtype == torch.float32 and delta.numel() == B * Hq * Sq):
        raise RuntimeError("attn_bwd_chunks: delta must be contiguous fp32 [B,H,S]")
    given = [t for t in (dks or []) if t is not None]
    dkv_dt, dks_arr = PICO_F32, None
    if given:
        g0 = given[0]
        for a, b_ in zip(dks, dvs):
            if (a is None) != (b_ is None):
                raise RuntimeError("attn_bwd_chunks: dk and dv of a chunk must be given together")
            if a is not None and (a.dtype != g0.dtype or b_.dtype != g0.dtype or a.stride() != g0.stride() or b_.stride() != g0.stride()
                                  or a.stride(-1) != 1 or a.shape != ks[0].shape or not a.is_cuda or not b_.is_cuda):
                raise RuntimeError("attn_bwd_chunks: all dk / dv buffers must share dtype and strides (unit D stride) and have the chunks' shape")
        dkv_dt = _dt(g0, "dk/dv")
        dks_arr = (ctypes.c_int64 * 3)(*g0.stride()[:3])
    if dq is not None and dq.stride(-1) != 1:
        raise RuntimeError("attn_bwd_chunks: dq needs a unit D stride")
    dqs = (ctypes.c_int64 * 3)(*(dq.stride()[:3] if dq is not None else (0, 0, 0)))
    finals = [t for t in (dk_finals or []) if t is not None]
    if finals:
        f0 = finals[0]
        for a, b_ in zip(dk_finals, dv_finals):
            if (a is None) != (b_ is None):
                raise RuntimeError("attn_bwd_chunks: dk_final and dv_final of a chunk must be given together")
            if a is not None and (a.dtype != torch.bfloat16 or b_.dtype != torch.bfloat16 or a.stride() != f0.stride()
                                  or b_.stride() != f0.stride() or a.stride(-1) != 1 or a.shape != ks[0].shape
                                  or not a.is_cuda or not b_.is_cuda):
                raise RuntimeError("attn_bwd_chunks: dk_final / dv_final must be bf16 buffers of the chunks' shape that share "
                                   "one stride triple (unit D stride)")
    d = _chunk_desc(q, ks, vs, dout, sm_scale, causal, q_offset)
    kv = _kv_chunks(ks, vs, dks if given else None, dvs, dkv_accumulate, dk_finals if finals else None, dv_finals)
    tables = ctypes.byref(_rope_tables(*rope)) if rope is not None else None
    check(_lib.lib().pico_attn_bwd_chunks(ctypes.byref(d), _ptr(q), ctypes.byref(kv), _ptr(dout), _ptr(out),
                                          _dt(out, "out") if out is not None else PICO_BF16, _ptr(lse.contiguous()), _ptr(delta),
                                          _ptr(dq), dqs, _dt(dq, "dq") if dq is not None else PICO_F32, int(dq_accumulate),
                                          dks_arr, dkv_dt, tables, int(q_pos_offset), int(k_pos_offset), _stream()))
    return delta


def attn_bwd_preprocess(dout: torch.Tensor, out: torch.Tensor, dq_acc: Optional[torch.Tensor] = None,
                        delta: Optional[torch.Tensor] = None) -> torch.Tensor:
    """delta = sum(dout * out, -1) as fp32 [B,H,S]; zeroes dq_acc (fp32 contiguous [B,H,S,D]) if given."""
    _dev(dout, out, dq_acc)
    dout = _attn_in(dout, "dout")
    if out.stride() != dout.stride():
        out = _like_strided(out, dout)
    B, H, S, D = dout.shape
    if delta is None:
        delta = torch.empty(B, H, S, dtype=torch.float32, device=dout.device)
    elif not (delta.is_contiguous() and delta.dtype == torch.float32 and delta.numel() == B * H * S):
        raise RuntimeError("attn_bwd_preprocess: delta must be contiguous fp32 [B,H,S]")
    d = _desc(dout, dout, dout, dout, 1.0, False, 0)
    if dq_acc is not None and not (dq_acc.is_contiguous() and dq_acc.dtype == torch.float32):
        raise RuntimeError("attn_bwd_preprocess: dq_acc must be contiguous fp32")
    check(_lib.lib().pico_attn_bwd_preprocess(ctypes.byref(d), _ptr(dout), _ptr(out), _dt(out, "attn out"), _ptr(delta),
                                              _ptr(dq_acc), _stream()))
    return delta


def _like_strided(t: torch.Tensor, ref: torch.Tensor) -> torch.Tensor:
    """Copy of t laid out with ref's strides (so one stride triple describes both)."""
    r = torch.empty_strided(ref.shape, ref.stride(), dtype=t.dtype, device=t.device)
    r.copy_(t)
    return r


def attn_bwd(dout, q, k, v, lse, delta, sm_scale: float, causal: bool, q_offset: int = 0,
             dq: Optional[torch.Tensor] = None, dk: Optional[torch.Tensor] = None, dv: Optional[torch.Tensor] = None,
             dq_accumulate: bool = False, dkv_accumulate: bool = False, dq_dtype=torch.float32,
             dkv_dtype=torch.float32, dq_like: Optional[torch.Tensor] = None, want_dq: bool = True,
             want_dkv: bool = True, side_stream: Optional["torch.cuda.Stream"] = None,
             out: Optional[torch.Tensor] = None, dkv_like: Optional[torch.Tensor] = None):
    """Gradients of one attention block; returns (dq [B,Hq,Sq,D], dk, dv [B,Hkv,Sk,D]).

    Buffers that are passed in are written in place (fp32 ones can be accumulated into: the running dq of a
    rank and the travelling dk / dv of the ring); missing ones are allocated in the requested dtype, dq with
    the strides of `dq_like` if given, dk / dv with the strides of `dkv_like` (so that a gradient for a [B,H,S,D] view
    of [B,S,H,D] memory needs no layout copy on its way back).  want_dq / want_dkv = False skips that gradient.
    With `out` (the forward output) `delta` may be None or a buffer to fill: the row sums delta = sum_d dout * out are
    then computed inside the call (by the dQ kernel itself when out is bf16 and dq is wanted), as in the reference's
    ring_attention_backward, instead of by a separate attn_bwd_preprocess.
    With `side_stream` the dQ kernel is enqueued there and the dK/dV kernel on the current stream (the two are
    independent); the current stream waits for both.  Measured on MI355X it is a wash at the benchmark shape
    (+3 % on one box, -4 % on another: the fork / join costs what the overlapped tails save), so nothing in
    this package turns it on by default.
    """
    _dev(dout, q, k, v, lse, delta, dq, dk, dv, out)
    q, k, v, dout = _attn_in(q, "q"), _attn_in(k, "k"), _attn_in(v, "v"), _attn_in(dout, "dout")
    B, Hq, Sq, D = q.shape
    Hkv, Sk = k.size(1), k.size(2)
    if out is not None:
        if side_stream is not None:
            raise RuntimeError("attn_bwd: out= (delta computed by the dQ kernel) orders the two kernels; no side_stream")
        if out.stride() != dout.stride():
            out = _like_strided(out, dout)
        if delta is None:
            delta = torch.empty(B, Hq, Sq, dtype=torch.float32, device=q.device)
        elif not (delta.is_contiguous() and delta.dtype == torch.float32 and delta.numel() == B * Hq * Sq):
            raise RuntimeError("attn_bwd: delta must be contiguous fp32 [B,H,S]")
    elif delta is None:
        raise RuntimeError("attn_bwd: delta (or out, to compute it) is required")
    if dq is None and want_dq:
        if dq_accumulate:
            raise RuntimeError("attn_bwd: dq_accumulate=True needs an existing dq")
        if dq_like is not None and _dense(dq_like) and dq_like.stride(-1) == 1 and dq_like.shape == q.shape:
            dq = torch.empty_strided(q.shape, dq_like.stride(), dtype=dq_dtype, device=q.device)
        else:
            dq = torch.empty(B, Hq, Sq, D, dtype=dq_dtype, device=q.device)
    if (dk is None or dv is None) and want_dkv:
        if dkv_accumulate:
            raise RuntimeError("attn_bwd: dkv_accumulate=True needs existing dk / dv")
        if dkv_like is not None and _dense(dkv_like) and dkv_like.stride(-1) == 1 and dkv_like.shape == k.shape:
            dk = torch.empty_strided(k.shape, dkv_like.stride(), dtype=dkv_dtype, device=q.device)
            dv = torch.empty_strided(k.shape, dkv_like.stride(), dtype=dkv_dtype, device=q.device)
        else:
            dk = torch.empty(B, Hkv, Sk, D, dtype=dkv_dtype, device=q.device)
            dv = torch.empty(B, Hkv, Sk, D, dtype=dkv_dtype, device=q.device)
    if not want_dq:
        dq = None
    if not want_dkv:
        dk = dv = None
    if dk is not None and (dk.dtype != dv.dtype or dk.stride() != dv.stride() or dk.stride(-1) != 1):
        raise RuntimeError("attn_bwd: dk and dv must share dtype and strides, with a unit D stride")
    if dq is not None and dq.stride(-1) != 1:
        raise RuntimeError("attn_bwd: dq needs a unit D stride")
    if lse.dtype != torch.float32 or delta.dtype != torch.float32:
        raise RuntimeError("attn_bwd: lse and delta must be fp32")
    d = _desc(q, k, v, dout, sm_scale, causal, q_offset)
    dqs = (ctypes.c_int64 * 3)(*(dq.stride()[:3] if dq is not None else (0, 0, 0)))
    dks = (ctypes.c_int64 * 3)(*(dk.stride()[:3] if dk is not None else (0, 0, 0)))
    lse_c, delta_c = lse.contiguous(), delta.contiguous()

    def launch(dq_, dk_, dv_):
        if out is not None:
            check(_lib.lib().pico_attn_bwd_fused(ctypes.byref(d), _ptr(q), _ptr(k), _ptr(v), _ptr(dout), _ptr(out),
                                                 _dt(out, "out"), _ptr(lse_c), _ptr(delta_c), _ptr(dq_), dqs,
                                                 _dt(dq, "dq") if dq is not None else PICO_F32, int(dq_accumulate),
                                                 _ptr(dk_), _ptr(dv_), dks,
                                                 _dt(dk, "dk/dv") if dk is not None else PICO_F32, int(dkv_accumulate),
                                                 _stream()))
            return
        check(_lib.lib().pico_attn_bwd(ctypes.byref(d), _ptr(q), _ptr(k), _ptr(v), _ptr(dout), _ptr(lse_c), _ptr(delta_c),
                                       _ptr(dq_), dqs, _dt(dq, "dq") if dq is not None else PICO_F32, int(dq_accumulate),
                                       _ptr(dk_), _ptr(dv_), dks, _dt(dk, "dk/dv") if dk is not None else PICO_F32,
                                       int(dkv_accumulate), _stream()))

    if side_stream is not None and dq is not None and dk is not None:
        cur = torch.cuda.current_stream()
        side_stream.wait_stream(cur)
        with torch.cuda.stream(side_stream):
            launch(dq, None, None)
        launch(None, dk, dv)
        cur.wait_stream(side_stream)
    else:
        launch(dq, dk, dv)
    return dq, dk, dv


def convert_f32(src: torch.Tensor, dtype, like: Optional[torch.Tensor] = None, bshd: bool = False,
                strides=None) -> torch.Tensor:
    """fp32 contiguous [B,H,S,D] -> dtype; laid out like `like` (same strides) or with the given `strides` (of a
    dense layout with a unit D stride), as a view over [B,S,H,D] memory (bshd=True), or contiguous."""
    _dev(src, like)
    if src.dtype != torch.float32 or not src.is_contiguous() or src.dim() != 4:
        raise RuntimeError("convert_f32: src must be a contiguous fp32 [B,H,S,D] tensor")
    B, H, S, D = src.shape
    if bshd:
        dst = empty_bshd(B, H, S, D, dtype, src.device)
    elif strides is not None:
        dst = torch.empty_strided(src.shape, tuple(strides), dtype=dtype, device=src.device)
        if dst.stride(-1) != 1 or not _dense(dst):
            raise RuntimeError("convert_f32: strides must describe a dense layout with a unit D stride")
    elif like is not None and _dense(like) and like.stride(-1) == 1:
        dst = torch.empty_strided(src.shape, like.stride(), dtype=dtype, device=src.device)
    else:
        dst = torch.empty(src.shape, dtype=dtype, device=src.device)
    check(_lib.lib().pico_convert_f32(_ptr(src), _ptr(dst), B, H, S, D, dst.stride(0), dst.stride(1), dst.stride(2),
                                      _DT[dtype], _stream()))
    return dst


def adamw_(param_lp: Optional[torch.Tensor], master: torch.Tensor, grad: torch.Tensor, exp_avg: torch.Tensor,
           exp_avg_sq: torch.Tensor, step: int, lr: float, beta1: float = 0.9, beta2: float = 0.999, eps: float = 1e-8,
           weight_decay: float = 0.01, grad_scale: float = 1.0) -> None:
    """In-place AdamW step on fp32 (master, exp_avg, exp_avg_sq) from a bf16 / fp32 gradient; rewrites the bf16
    parameter `param_lp` (if given) from the new master weight.  `step` counts from 1."""
    _dev(param_lp, master, grad, exp_avg, exp_avg_sq)
    n = master.numel()
    for t, what in ((master, "master"), (exp_avg, "exp_avg"), (exp_avg_sq, "exp_avg_sq")):
        if t.dtype != torch.float32 or not t.is_contiguous() or t.numel() != n:
            raise RuntimeError(f"adamw_: {what} must be a contiguous fp32 tensor of {n} elements")
    if not grad.is_contiguous() or grad.numel() != n:
        grad = grad.contiguous()
        if grad.numel() != n:
            raise RuntimeError("adamw_: grad has the wrong number of elements")
    if param_lp is not None and (param_lp.dtype != torch.bfloat16 or not param_lp.is_contiguous() or param_lp.numel() != n):
        raise RuntimeError("adamw_: param_lp must be a contiguous bf16 tensor of the same size")
    check(_lib.lib().pico_adamw(_ptr(param_lp), _ptr(master), _ptr(grad), _dt(grad, "grad"), _ptr(exp_avg), _ptr(exp_avg_sq),
                                n, float(lr), float(beta1), float(beta2), float(eps), float(weight_decay), int(step),
                                float(grad_scale), _stream()))


def adamw_lp_(param: torch.Tensor, grad: torch.Tensor, exp_avg: torch.Tensor, exp_avg_sq: torch.Tensor, step: int,
              lr: float, beta1: float = 0.9, beta2: float = 0.999, eps: float = 1e-8, weight_decay: float = 0.01,
              grad_scale: float = 1.0) -> None:
    """In-place AdamW step on a bf16 parameter (no master copy) with fp32 moments, or with bf16 moments (the state
    torch.optim.AdamW holds for a bf16 model); fp32 arithmetic, one rounding per stored value.  `step` counts from 1."""
    _dev(param, grad, exp_avg, exp_avg_sq)
    n = param.numel()
    if param.dtype != torch.bfloat16 or not param.is_contiguous():
        raise RuntimeError("adamw_lp_: param must be a contiguous bf16 tensor")
    sdt = exp_avg.dtype
    for t, what in ((exp_avg, "exp_avg"), (exp_avg_sq, "exp_avg_sq")):
        if t.dtype != sdt or sdt not in _DT or not t.is_contiguous() or t.numel() != n:
            raise RuntimeError(f"adamw_lp_: {what} must be a contiguous bf16 or fp32 tensor of {n} elements")
    if grad.numel() != n:
        raise RuntimeError("adamw_lp_: grad has the wrong number of elements")
    grad = grad.contiguous()
    check(_lib.lib().pico_adamw_lp(_ptr(param), _ptr(grad), _dt(grad, "grad"), _ptr(exp_avg), _ptr(exp_avg_sq), n,
                                   _dt(param, "param"), _DT[sdt], float(lr), float(beta1), float(beta2), float(eps),
                                   float(weight_decay), int(step), float(grad_scale), _stream()))


class AdamWMultiPlan:
    """The AdamW step for a fixed list of tensors in as few launches as they fit (48 tensors each).  Weights, moments
    and sizes are checked and their pointer tables built once; a step only fills in the gradients' addresses, so its
    host cost is a fraction of a millisecond for a few hundred tensors.  All weights share one dtype and both moments
    of all tensors another: fp32 weights with fp32 moments (master weights; `param_lps` optionally lists the bf16
    parameters to rewrite, None entries allowed), or bf16 weights (the parameters themselves; `param_lps` must be None)
    with fp32 or bf16 moments.  The plan keeps the tensors alive."""

    def __init__(self, weights, exp_avgs, exp_avg_sqs, param_lps=None):
        count = len(weights)
        if count == 0 or not (len(exp_avgs) == len(exp_avg_sqs) == count) or (param_lps is not None and len(param_lps) != count):
            raise RuntimeError("adamw_multi_: the lists must have one entry per tensor (and at least one)")
        wdt, sdt = weights[0].dtype, exp_avgs[0].dtype
        for i in range(count):
            w, m, v = weights[i], exp_avgs[i], exp_avg_sqs[i]
            _dev(w, m, v)
            n = w.numel()
            for t, dt, what in ((w, wdt, "weight"), (m, sdt, "exp_avg"), (v, sdt, "exp_avg_sq")):
                if t.dtype != dt or not t.is_contiguous() or t.numel() != n:
                    raise RuntimeError(f"adamw_multi_: tensor {i}: {what} must be a contiguous {dt} tensor of {n} elements")
            if param_lps is not None and param_lps[i] is not None:
                lp = param_lps[i]
                _dev(lp)
                if lp.dtype != torch.bfloat16 or not lp.is_contiguous() or lp.numel() != n:
                    raise RuntimeError(f"adamw_multi_: tensor {i}: param_lp must be a contiguous bf16 tensor of {n} elements")
        self.count = count
        self._keep = (list(weights), list(exp_avgs), list(exp_avg_sqs), list(param_lps) if param_lps is not None else None)
        self._arr = ctypes.c_void_p * count
        table = lambda ts: self._arr(*[t.data_ptr() if t is not None else None for t in ts])
        self._w, self._m, self._v = table(weights), table(exp_avgs), table(exp_avg_sqs)
        self._lp = table(param_lps) if param_lps is not None else None
        self._numel = [w.numel() for w in weights]
        self._sizes = (ctypes.c_int64 * count)(*self._numel)
        self._weight_dt, self._state_dt = _dt(weights[0], "weight"), _dt(exp_avgs[0], "exp_avg")

    def step(self, grads, step: int, lr: float, beta1: float = 0.9, beta2: float = 0.999, eps: float = 1e-8,
             weight_decay: float = 0.01, grad_scale: float = 1.0) -> None:
        if len(grads) != self.count:
            raise RuntimeError("adamw_multi_: the lists must have one entry per tensor")
        gdt = grads[0].dtype
        keep = []   # contiguous copies of gradients must outlive the launch call
        g_arr = self._arr()
        for i, g in enumerate(grads):
            if not g.is_cuda:
                _dev(g)
            if g.dtype != gdt or g.numel() != self._numel[i]:
                raise RuntimeError(f"adamw_multi_: tensor {i}: grad must have dtype {gdt} and {self._numel[i]} elements")
            if not g.is_contiguous():
                g = g.contiguous()
                keep.append(g)
            g_arr[i] = g.data_ptr()
        check(_lib.lib().pico_adamw_multi(self.count, self._w, self._lp, g_arr, self._m, self._v, self._sizes,
                                          self._weight_dt, self._state_dt, _dt(grads[0], "grad"), float(lr), float(beta1), float(beta2),
                                          float(eps), float(weight_decay), int(step), float(grad_scale), _stream()))


def adamw_multi_(weights, grads, exp_avgs, exp_avg_sqs, step: int, lr: float, beta1: float = 0.9, beta2: float = 0.999,
                 eps: float = 1e-8, weight_decay: float = 0.01, grad_scale: float = 1.0, param_lps=None) -> None:
    """One AdamW step for a list of tensors (see AdamWMultiPlan, which a training loop should build once)."""
    if len(weights) == 0 and len(grads) == 0:
        return
    AdamWMultiPlan(weights, exp_avgs, exp_avg_sqs, param_lps).step(grads, step, lr, beta1, beta2, eps, weight_decay, grad_scale)


def _ce_check(logits: torch.Tensor, targets: torch.Tensor):
    _dev(logits, targets)
    if logits.dim() != 2 or logits.stride(1) != 1:
        raise RuntimeError("cross_entropy: logits must be [rows, vocab] with a unit stride on vocab")
    if targets.dtype != torch.int64 or not targets.is_contiguous() or targets.numel() != logits.size(0):
        raise RuntimeError("cross_entropy: targets must be a contiguous int64 tensor with one entry per row")


def cross_entropy_fwd(logits: torch.Tensor, targets: torch.Tensor, ignore_index: int = -100):
    """Per-row loss and logsumexp, both fp32 [rows]."""
    _ce_check(logits, targets)
    rows, vocab = logits.shape
    loss = torch.empty(rows, dtype=torch.float32, device=logits.device)
    lse = torch.empty(rows, dtype=torch.float32, device=logits.device)
    check(_lib.lib().pico_cross_entropy_fwd(_ptr(logits), _ptr(targets), _ptr(loss), _ptr(lse), rows, vocab,
                                            logits.stride(0) if rows else vocab, ignore_index, _dt(logits, "logits"), _stream()))
    return loss, lse


def cross_entropy_bwd(logits: torch.Tensor, targets: torch.Tensor, lse: torch.Tensor, scale: torch.Tensor,
                      ignore_index: int = -100, inplace: bool = False) -> torch.Tensor:
    """dlogits = (softmax(logits) - onehot(targets)) * scale, scale a one-element fp32 tensor on the device."""
    _ce_check(logits, targets)
    _dev(lse, scale)
    if scale.dtype != torch.float32 or scale.numel() != 1 or lse.dtype != torch.float32 or not lse.is_contiguous():
        raise RuntimeError("cross_entropy_bwd: lse must be contiguous fp32 [rows], scale one fp32 element")
    rows, vocab = logits.shape
    # same row pitch as the logits (a view into a padded buffer keeps its 16-byte-aligned rows)
    out = logits if inplace else torch.empty_strided(logits.shape, logits.stride(), dtype=logits.dtype, device=logits.device)
    check(_lib.lib().pico_cross_entropy_bwd(_ptr(logits), _ptr(targets), _ptr(lse), _ptr(scale), _ptr(out), rows, vocab,
                                            logits.stride(0) if rows else vocab, out.stride(0) if rows else vocab,
                                            ignore_index, _dt(logits, "logits"), _stream()))
    return out

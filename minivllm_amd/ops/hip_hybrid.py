"""ctypes bindings for ``_hip_hybrid.so`` (``csrc/hybrid``): the gfx950 kernels of hybrid
decoders.  Same conventions as ``ops.hip``: raw device pointers, element strides, the current
HIP stream (so calls made during graph capture become graph nodes), no PyTorch fallback.  The
library is built on first use when it is missing (a few seconds, hipcc only).  Tensors are
bfloat16 or float32 (``dt`` 0 / 2); fp32 tensors (stream, state, router, norm weights) are always
fp32.  Function signatures mirror ``ops.torch_seqmix``.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional

import torch

_LIB_PATH = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))),
                         "_hip_hybrid.so")
if not os.path.exists(_LIB_PATH):
    from minivllm_amd import build as _build
    _build.build_hip_group("hybrid", verbose=False)
_lib = ctypes.CDLL(_LIB_PATH)

_L, _I, _F, _P = ctypes.c_long, ctypes.c_int, ctypes.c_float, ctypes.c_void_p


def _sig(name, *argtypes):
    f = getattr(_lib, name)
    f.argtypes = list(argtypes)
    f.restype = ctypes.c_int
    return f


_embed = _sig("hyb_embed_sum", _P, _P, _P, _P, _P, _L, _I, _I, _P)
_norm = _sig("hyb_offset_rms_norm", _P, _P, _P, _L, _I, _F, _I, _P)
_post = _sig("hyb_post_norm_residual", _P, _L, _P, _P, _P, _P, _L, _I, _F, _I, _P)
_rope = _sig("hyb_pair_rope_mix_store", _P, _P, _P, _L, _P, _P, _I, _P, _P, _I, _P, _P, _P, _L,
             _I, _I, _I, _I, _I, _P)
_ghn = _sig("hyb_gated_head_norm", _P, _P, _P, _L, _P, _L, _I, _I, _F, _I, _P)
_route = _sig("hyb_grouped_route", _P, _P, _P, _L, _I, _I, _I, _I, _I, _I, _P)
_gelu = _sig("hyb_gelu_route_scale", _P, _P, _P, _L, _I, _I, _I, _P)
_attn = _sig("hyb_sink_attention_rows", _P, _L, _L, _P, _P, _P, _I, _I, _P, _P, _I, _P, _P, _L, _P,
             _F, _L, _I, _I, _I, _I, _I, _I, _P)
_tiles = _sig("hyb_sink_attention_tiles", _P, _L, _L, _P, _P, _P, _I, _I, _P, _P, _P, _P, _L, _P, _F,
              _I, _I, _I, _I, _I, _I, _I, _I, _P)
_tiles_ok = _lib.hyb_sink_attention_tiles_ok
_tiles_ok.argtypes = [_I, _I]
_tiles_ok.restype = _I
_split = _sig("hyb_sink_attention_split", _P, _L, _L, _P, _P, _P, _I, _I, _P, _P, _P, _L, _P, _P, _F,
              _I, _I, _I, _I, _I, _I, _I, _P)
_split_ok = _lib.hyb_sink_attention_split_ok
_split_ok.argtypes = [_I, _I]
_split_ok.restype = _I
_prep = _sig("hyb_delta_prepare", _P, _L, _I, _I, _P, _I, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P,
             _P, _P, _L, _I, _I, _I, _I, _I, _I, _P)
_scan = _sig("hyb_delta_scan", _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P)

_DT = {torch.bfloat16: 0, torch.float32: 2}


def _dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise TypeError(f"hybrid kernels take bfloat16 / float32 activations, got {t.dtype}")


def _stream() -> int:
    return torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())


def _check(rc: int, name: str) -> None:
    if rc != 0:
        raise RuntimeError(f"{name} failed (code {rc}): shape outside the kernel's range or a "
                           f"HIP launch error")


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _f32(t: torch.Tensor) -> torch.Tensor:
    assert t.dtype == torch.float32 and t.is_contiguous(), "fp32 contiguous tensor expected"
    return t


def _i32(t: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    if t is None:
        return None
    assert t.dtype == torch.int32 and t.is_contiguous()
    return t


def _rows(t: torch.Tensor) -> int:
    """Row stride (elements) of a [T, ...] view whose trailing dims are dense."""
    assert t.stride(-1) == 1
    return t.stride(0) if t.shape[0] > 1 else int(t.stride(0) or t[0].numel())


# ------------------------------------------------------------------ embedding + norms
def embed_sum(ids, aux_rows, table, aux_table):
    T, W = ids.shape[0], table.shape[1]
    x = torch.empty((T, W), dtype=torch.float32, device=table.device)
    _check(_embed(_ptr(_i32(ids)), _ptr(_i32(aux_rows)) if aux_table is not None else None,
                  table.data_ptr(), _ptr(aux_table), x.data_ptr(), T, W, _dt(table), _stream()),
           "embed_sum")
    return x


def offset_rms_norm(x, w, eps, out_dtype):
    x = _f32(x)
    T, W = x.shape
    out = torch.empty((T, W), dtype=out_dtype, device=x.device)
    _check(_norm(x.data_ptr(), _f32(w).data_ptr(), out.data_ptr(), T, W, eps, _dt(out), _stream()),
           "offset_rms_norm")
    return out


def post_norm_residual(y, wb, x, eps, w_next, out_dtype):
    x = _f32(x)
    T, W = x.shape
    assert y.shape == x.shape and y.stride(-1) == 1 and y.dtype == out_dtype
    h = torch.empty((T, W), dtype=out_dtype, device=x.device) if w_next is not None else None
    _check(_post(y.data_ptr(), y.stride(0), _f32(wb).data_ptr(), x.data_ptr(),
                 _ptr(w_next), _ptr(h), T, W, eps, _dt(y), _stream()), "post_norm_residual")
    return h


# ------------------------------------------------------------------ rotation, value mix, store
def pair_rope_mix_store(q, k, v, positions, cos_sin, rot_dims, v_first, lam, v_mode,
                        k_cache, v_cache, slot_mapping):
    T, H, D = q.shape
    G, E = v.shape[1], v.shape[2]
    rs = q.stride(0)
    assert (T == 1 or (k.stride(0) == rs and v.stride(0) == rs)) and q.stride(1) == D \
        and k.stride(1) == D and v.stride(1) == E and q.stride(2) == 1, \
        "q / k / v must be views of one projection output"
    if k_cache is not None:
        assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.dtype == q.dtype
    if rot_dims:
        assert cos_sin.shape[1] == rot_dims and cos_sin.dtype == torch.float32
    if v_mode:
        assert v_first is not None and v_first.is_contiguous() and v_first.dtype == q.dtype \
            and v_first.numel() == T * G * E
    _check(_rope(q.data_ptr(), k.data_ptr(), v.data_ptr(), rs, _i32(positions).data_ptr(),
                 _ptr(cos_sin) if rot_dims else None, rot_dims, _ptr(v_first) if v_mode else None,
                 _f32(lam).data_ptr(), v_mode, _ptr(k_cache), _ptr(v_cache), _ptr(_i32(slot_mapping)),
                 T, H, G, D, E, _dt(q), _stream()), "pair_rope_mix_store")


# ------------------------------------------------------------------ attention with a sink
def _attention_rows(q, k_cache, v_cache, block_tables, row_seq, lens, len_add, scale, sink, gate, out,
                    seq_base=0):
    T, H, D = q.shape
    G, E = k_cache.shape[2], v_cache.shape[3]
    assert q.stride(2) == 1 and out.is_contiguous() and out.shape == (T, H, E) and out.dtype == q.dtype
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.dtype == q.dtype
    assert block_tables.dtype == torch.int32 and block_tables.stride(1) == 1
    if gate is not None:
        assert gate.stride(1) == 1 and gate.dtype == q.dtype
    _check(_attn(q.data_ptr(), q.stride(0), q.stride(1), k_cache.data_ptr(), v_cache.data_ptr(),
                 block_tables.data_ptr(), block_tables.stride(0), k_cache.shape[1],
                 _ptr(_i32(row_seq)), _i32(lens).data_ptr(), len_add, _f32(sink).data_ptr(),
                 _ptr(gate), gate.stride(0) if gate is not None else 0, out.data_ptr(), scale, T,
                 H, G, D, E, seq_base, _dt(q), _stream()), "sink_attention")
    return out


def sink_attention_step(q, k_cache, v_cache, block_tables, row_seq, positions, scale, sink, gate, out,
                        seq_base=0):
    """Rows of a prefill-form step, one workgroup per row: row t belongs to sequence
    ``row_seq[t]`` (< ``seq_base``: skipped), whose block table is row ``row_seq[t] - seq_base``
    of ``block_tables``, and sees ``positions[t] + 1`` keys."""
    return _attention_rows(q, k_cache, v_cache, block_tables, row_seq, positions, 1, scale, sink,
                           gate, out, seq_base)


def sink_attention_prefill(q, k_cache, v_cache, cu_q, cu_k, block_tables, scale, sink, gate, out,
                           positions=None, max_q=None, row_seq=None, first_seq=0):
    """The prompt portions of a step: sequence b owns rows cu_q[b] .. cu_q[b+1] (absolute rows
    of q / out / positions) and block table row b.  Runs the matrix-core tile kernel (fp32
    scores, weights and sums); head sizes it has no instance for go row by row.  ``cu_k`` is
    not needed (a row's context is its position + 1)."""
    T, H, D = q.shape
    G, E = k_cache.shape[2], v_cache.shape[3]
    nseq = cu_q.shape[0] - 1
    assert positions is not None, "the GPU form takes the rows' positions"
    if not _tiles_ok(D, E):
        assert row_seq is not None
        # ``first_seq``: number of the step's sequences ahead of these (its decode riders)
        return sink_attention_step(q, k_cache, v_cache, block_tables, row_seq, positions, scale,
                                   sink, gate, out, seq_base=first_seq)
    if max_q is None:
        max_q = int((cu_q[1:] - cu_q[:-1]).max())
    assert q.stride(2) == 1 and out.is_contiguous() and out.shape == (T, H, E) and out.dtype == q.dtype
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.dtype == q.dtype
    assert block_tables.dtype == torch.int32 and block_tables.stride(1) == 1
    if gate is not None:
        assert gate.stride(1) == 1 and gate.dtype == q.dtype
    _check(_tiles(q.data_ptr(), q.stride(0), q.stride(1), k_cache.data_ptr(), v_cache.data_ptr(),
                  block_tables.data_ptr(), block_tables.stride(0), k_cache.shape[1],
                  _i32c(cu_q).data_ptr(), _i32(positions).data_ptr(), _f32(sink).data_ptr(),
                  _ptr(gate), gate.stride(0) if gate is not None else 0, out.data_ptr(), scale,
                  nseq, 0, max_q, H, G, D, E, _dt(q), _stream()), "sink_attention_prefill")
    return out


def _i32c(t):
    assert t.dtype == torch.int32 and t.stride(0) == 1
    return t


def decode_splits(batch: int, kv_heads: int, heads: int, max_context_len) -> int:
    """Workgroups per (sequence, KV head group) of the split decode kernel: enough to fill the
    256 CUs several times over, each with at least 128 keys of the longest context."""
    groups = kv_heads * -(-(heads // kv_heads) // 4)
    want = max(1, 2048 // max(batch * groups, 1))
    room = max(1, (int(max_context_len) + 127) // 128) if max_context_len else 8
    return max(1, min(16, want, room))


def sink_attention_decode(q, k_cache, v_cache, block_tables, context_lens, scale, sink, gate, out,
                          max_context_len=None):
    """Single next tokens: row b is sequence b with ``context_lens[b]`` keys.  Head sizes the
    split-context kernel has an instance for (D in 64 / 128 / 256, E in 64 / 128) stream K / V
    rows with coalesced 16-byte loads over several workgroups per sequence and are merged by a
    second small kernel; other sizes go through the row kernel."""
    B, H, D = q.shape
    G, E = k_cache.shape[2], v_cache.shape[3]
    es = q.element_size()
    if (_split_ok(D, E) and q.stride(2) == 1 and q.stride(1) == D and q.data_ptr() % 16 == 0
            and (B == 1 or (q.stride(0) * es) % 16 == 0) and k_cache.is_contiguous()
            and v_cache.is_contiguous() and out.is_contiguous()):
        splits = decode_splits(B, G, H, max_context_len)
        ws = torch.empty((B * H * splits * (E + 2),), dtype=torch.float32, device=q.device)
        if gate is not None:
            assert gate.stride(1) == 1 and gate.dtype == q.dtype
        _check(_split(q.data_ptr(), q.stride(0) if B > 1 else H * D, q.stride(1), k_cache.data_ptr(),
                      v_cache.data_ptr(), block_tables.data_ptr(), block_tables.stride(0),
                      k_cache.shape[1], _i32c(context_lens).data_ptr(), _f32(sink).data_ptr(),
                      _ptr(gate), gate.stride(0) if gate is not None else 0, out.data_ptr(),
                      ws.data_ptr(), scale, B, H, G, D, E, splits, _dt(q), _stream()),
               "sink_attention_decode")
        return out
    return _attention_rows(q, k_cache, v_cache, block_tables, None, context_lens, 0, scale, sink,
                           gate, out)


# ------------------------------------------------------------------ gated delta rule
def delta_prepare(q, k, v, b, a, conv_w, a_log, dt_bias, conv_state, cu_q, positions, slots,
                  row_seq):
    T, G, D = q.shape
    H, E = v.shape[1], v.shape[2]
    rs = q.stride(0)
    base = q.data_ptr()
    es = q.element_size()
    # q, k, v are the first three column blocks of one projection output, b and a views of it
    assert k.data_ptr() == base + G * D * es and v.data_ptr() == base + 2 * G * D * es
    assert T == 1 or (k.stride(0) == rs and v.stride(0) == rs and b.stride(0) == rs
                      and a.stride(0) == rs)
    b_off, a_off = (b.data_ptr() - base) // es, (a.data_ptr() - base) // es
    dev = q.device
    taps = _f32(conv_w).shape[1]
    assert conv_w.shape[0] == 2 * G * D + H * E
    f = dict(dtype=torch.float32, device=dev)
    qn, kn = torch.empty((T, G, D), **f), torch.empty((T, G, D), **f)
    vv, beta, decay = torch.empty((T, H, E), **f), torch.empty((T, H), **f), torch.empty((T, H), **f)
    if cu_q is not None:
        assert row_seq is not None, "prefill-form steps pass the sequence of each row"
    B = slots.shape[0]
    _check(_prep(base, rs, b_off, a_off, conv_w.data_ptr(), taps, _f32(a_log).data_ptr(),
                 _f32(dt_bias).data_ptr(), _f32(conv_state).data_ptr(), _ptr(_i32(cu_q)),
                 _i32(positions).data_ptr(), _i32(slots).data_ptr(),
                 _ptr(_i32(row_seq)) if cu_q is not None else None, qn.data_ptr(), kn.data_ptr(),
                 vv.data_ptr(), beta.data_ptr(), decay.data_ptr(), T, B, H, G, D, E, _dt(q),
                 _stream()), "delta_prepare")
    return qn, kn, vv, beta, decay


def delta_scan(qn, kn, vv, beta, decay, state, cu_q, positions, slots):
    T, G, D = qn.shape
    H, E = vv.shape[1], vv.shape[2]
    assert state.shape[1:] == (H, D, E)
    o = torch.zeros((T, H, E), dtype=torch.float32, device=qn.device)
    _check(_scan(qn.data_ptr(), kn.data_ptr(), vv.data_ptr(), beta.data_ptr(), decay.data_ptr(),
                 _f32(state).data_ptr(), _ptr(_i32(cu_q)), _i32(positions).data_ptr(),
                 _i32(slots).data_ptr(), o.data_ptr(), slots.shape[0], H, G, D, E, _stream()),
           "delta_scan")
    return o


def gated_head_norm(o, w, gate, eps, out_dtype):
    T, H, E = o.shape
    assert gate.stride(-1) == 1 and gate.dtype == out_dtype
    out = torch.empty((T, H, E), dtype=out_dtype, device=o.device)
    _check(_ghn(_f32(o).data_ptr(), _f32(w).data_ptr(), gate.data_ptr(), gate.stride(0),
                out.data_ptr(), T, H, E, eps, _dt(out), _stream()), "gated_head_norm")
    return out


# ------------------------------------------------------------------ grouped expert routing
def grouped_route(h, router_w, top, groups, keep):
    T, W = h.shape
    NE = router_w.shape[0]
    assert h.is_contiguous()
    dense = torch.empty((T, NE), dtype=torch.float32, device=h.device)
    _check(_route(h.data_ptr(), _f32(router_w).data_ptr(), dense.data_ptr(), T, W, NE, top, groups,
                  keep, _dt(h), _stream()), "grouped_route")
    return dense


def gelu_route_scale(up, dense, ff, out_dtype):
    T = up.shape[0]
    NE = dense.shape[1]
    assert up.is_contiguous() and up.dtype == out_dtype and up.shape[1] == NE * ff
    act = torch.empty_like(up)
    _check(_gelu(up.data_ptr(), _f32(dense).data_ptr(), act.data_ptr(), T, NE, ff, _dt(up),
                 _stream()), "gelu_route_scale")
    return act

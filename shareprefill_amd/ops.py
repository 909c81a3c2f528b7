"""Torch-tensor front ends of the C-ABI entry points (include/shareprefill_hip.h).

Each function validates shapes on the host, allocates the outputs with torch, and enqueues the HIP
kernels on torch's current stream.  Tensors follow the library's conventions: token-major or
head-major q/k/v given as [H, N, D] views with arbitrary token / head strides and contiguous head_dim.
"""

from __future__ import annotations

import ctypes as C
from typing import Optional

import torch

from . import _lib
from ._lib import ClusterStateStruct


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream_handle(device=None) -> int:
    """Raw handle of torch's current stream on the current device.  Every kernel of the path is launched on it, so
    tensors of another device are refused rather than launched on a stream that does not belong to them.  Called a
    dozen times per layer: the raw accessors cost a fraction of torch.cuda.current_stream()."""
    if _raw_stream is not None and _raw_device is not None:
        cur = _raw_device()
        if device is not None and device.index is not None and device.index != cur:
            raise ValueError(f"tensors live on cuda:{device.index} but the current device is cuda:{cur}; "
                             "run the call under torch.cuda.device(...)")
        return int(_raw_stream(cur))
    return int(torch.cuda.current_stream(device).cuda_stream)


def _stream(device=None) -> C.c_void_p:
    return C.c_void_p(_stream_handle(device))


def _ptr(t: Optional[torch.Tensor]) -> C.c_void_p:
    return C.c_void_p(0 if t is None else t.data_ptr())


def _check_hnd(t: torch.Tensor, name: str):
    if t.dim() != 3:
        raise ValueError(f"{name} must be [H, N, D], got {tuple(t.shape)}")
    if t.dtype != torch.bfloat16:
        raise AssertionError(f"{name} must be bfloat16, got {t.dtype}")
    if not t.is_cuda:
        raise ValueError(f"{name} must live on the GPU")
    if t.stride(2) != 1:
        raise ValueError(f"{name} must have a contiguous head_dim axis")


def pool_avg(x: torch.Tensor, block_size: int, tail_mode: int = _lib.SP_POOL_TAIL_TRUE_LENGTH,
             head_enable: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x: bf16 [H, N, D] view -> bf16 [nb, H, D] block means (reference: triton_bnhd_pool, attn/utils.py:211-261)."""
    lib = _lib.load()
    _check_hnd(x, "x")
    h, n, d = x.shape
    nb = -(-n // block_size)
    if out is None:
        out = torch.empty(nb, h, d, dtype=torch.bfloat16, device=x.device)
    st = lib.sp_pool_avg_bf16(_ptr(x), _ptr(out), n, h, d, x.stride(1), x.stride(0), block_size, tail_mode,
                              _ptr(head_enable), _stream(x.device))
    _lib.check(st, "sp_pool_avg_bf16")
    return out


def pool(x: torch.Tensor, block_size: int, pool_type: str) -> torch.Tensor:
    """x: bf16 [H, N, D] view -> bf16 [nb, H, D], one of the reference kernel's pool types "avg", "max", "min",
    "maxabs", "sum" per block of block_size tokens (bnhd_pool_kernel, attn/utils.py:131-208)."""
    lib = _lib.load()
    _check_hnd(x, "x")
    if pool_type not in _lib.SP_POOL_TYPES:
        raise KeyError(pool_type)
    h, n, d = x.shape
    nb = -(-n // block_size)
    out = torch.empty(nb, h, d, dtype=torch.bfloat16, device=x.device)
    st = lib.sp_pool_bf16(_ptr(x), _ptr(out), n, h, d, x.stride(1), x.stride(0), block_size,
                          _lib.SP_POOL_TYPES[pool_type], _stream(x.device))
    _lib.check(st, "sp_pool_bf16")
    return out


_workspaces = {}


def _workspace(tag: str, nbytes: int, device) -> torch.Tensor:
    """Grow-only scratch buffers keyed by purpose, device AND stream (reused across layers).  Work on one stream is
    ordered, so consecutive calls may share a buffer; two streams of one device (two models, two threads) get
    buffers of their own and cannot race on the scheduler tickets or the repacked V they hold."""
    key = (tag, str(device), _stream_handle(device))
    buf = _workspaces.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=device)
        _workspaces[key] = buf
    return buf


def release_workspaces(device=None) -> None:
    """Drops the cached scratch buffers (all of them, or one device's).  Synchronise first: kernels still running
    on a buffer's stream keep using it."""
    for key in [k for k in _workspaces if device is None or k[1] == str(device)]:
        del _workspaces[key]


def lastq_scores(q: torch.Tensor, k: torch.Tensor, block_size: int, flags: int = _lib.SP_FLAG_LOGITS_BF16):
    """q [Hq,N,D], k [Hkv,N,D] -> (vert_tok [Hq,N], slash_tok [Hq,N], vert_blk [Hq,nb], slash_blk [Hq,nb]) fp32.

    Reference: attention_sharing.py:127-180 (Step A and the block sum-pool)."""
    lib = _lib.load()
    _check_hnd(q, "q")
    _check_hnd(k, "k")
    hq, n, d = q.shape
    hkv = k.shape[0]
    nb = -(-n // block_size)
    dev = q.device
    vert_tok = torch.empty(hq, n, dtype=torch.float32, device=dev)
    slash_tok = torch.empty(hq, n, dtype=torch.float32, device=dev)
    vert_blk = torch.empty(hq, nb, dtype=torch.float32, device=dev)
    slash_blk = torch.empty(hq, nb, dtype=torch.float32, device=dev)
    need = lib.sp_lastq_scores_workspace_bytes(n, hq, block_size)
    ws = _workspace("lastq", need, dev)
    st = lib.sp_lastq_scores_bf16(_ptr(q), _ptr(k), n, hq, hkv, d, q.stride(1), q.stride(0), k.stride(1), k.stride(0),
                                  block_size, flags, _ptr(ws), ws.numel(), _ptr(vert_tok), _ptr(slash_tok),
                                  _ptr(vert_blk), _ptr(slash_blk), _stream(dev))
    _lib.check(st, "sp_lastq_scores_bf16")
    return vert_tok, slash_tok, vert_blk, slash_blk


def cover_count(x: torch.Tensor, thr: float) -> torch.Tensor:
    """x fp32 [V, L] -> int32 [V] = count(cumsum(sort_desc(x)) <= thr) + 1 (attn/utils.py:47-50)."""
    lib = _lib.load()
    assert x.dtype == torch.float32 and x.dim() == 2 and x.is_contiguous() and x.is_cuda
    out = torch.empty(x.shape[0], dtype=torch.int32, device=x.device)
    ws = _workspace("cover_select", lib.sp_cover_select_workspace_bytes(x.shape[0]), x.device)
    _lib.check(lib.sp_cover_count(_ptr(x), x.shape[0], x.shape[1], thr, _ptr(out), _ptr(ws), ws.numel(), _stream(x.device)),
               "sp_cover_count")
    return out


def cover_budgets(vert_tok, slash_tok, block_size, pattern_threshold, min_blocks, max_blocks):
    """Per-head vertical / slash block budgets, int32 [Hq] each (attention_sharing.py:169-176)."""
    lib = _lib.load()
    assert vert_tok.is_contiguous() and slash_tok.is_contiguous() and vert_tok.dtype == torch.float32
    hq, n = vert_tok.shape
    nv = torch.empty(hq, dtype=torch.int32, device=vert_tok.device)
    ns = torch.empty(hq, dtype=torch.int32, device=vert_tok.device)
    ws = _workspace("cover_select", lib.sp_cover_select_workspace_bytes(2 * hq), vert_tok.device)
    st = lib.sp_cover_budgets(_ptr(vert_tok), _ptr(slash_tok), hq, n, block_size, pattern_threshold, min_blocks,
                              max_blocks, _ptr(nv), _ptr(ns), _ptr(ws), ws.numel(), _stream(vert_tok.device))
    _lib.check(st, "sp_cover_budgets")
    return nv, ns


def queryaware_test(q, kbar, vert_blk, block_size, queryaware_threshold, flags=_lib.SP_FLAG_LOGITS_BF16):
    """-> (avg_qk [Hq,nb] fp32, js_qa [Hq] fp32, use_qa [Hq] int32) (attention_sharing.py:193-202)."""
    lib = _lib.load()
    _check_hnd(q, "q")
    hq, n, d = q.shape
    nb, hkv, _ = kbar.shape
    assert kbar.is_contiguous() and kbar.dtype == torch.bfloat16 and vert_blk.is_contiguous()
    dev = q.device
    avg_qk = torch.empty(hq, nb, dtype=torch.float32, device=dev)
    js = torch.empty(hq, dtype=torch.float32, device=dev)
    use = torch.empty(hq, dtype=torch.int32, device=dev)
    st = lib.sp_queryaware_test_bf16(_ptr(q), _ptr(kbar), _ptr(vert_blk), n, hq, hkv, d, q.stride(1), q.stride(0),
                                     block_size, flags, queryaware_threshold, _ptr(avg_qk), _ptr(js), _ptr(use),
                                     _stream(dev))
    _lib.check(st, "sp_queryaware_test_bf16")
    return avg_qk, js, use


class ClusterState:
    """Device slabs of the cross-layer sharing state for C shared clusters (struct sp_cluster_state)."""

    def __init__(self, n_clusters: int, nb: int, device, keep_maps: bool = False):
        self.n_clusters, self.nb, self.nbw, self.device = n_clusters, nb, (nb + 63) // 64, device
        c = max(n_clusters, 1)
        # the pivots' block-average maps themselves (fp32 [C, nb, nb]), only when asked for
        self.avg_map = torch.empty(c, nb, nb, dtype=torch.float32, device=device) if keep_maps else None
        self.info = torch.zeros(c, 8, dtype=torch.int32, device=device)
        self.ratio = torch.zeros(c, dtype=torch.float64, device=device)
        self.vert = torch.zeros(c, nb, dtype=torch.float32, device=device)
        self.slash = torch.zeros(c, nb, dtype=torch.float32, device=device)
        self.cols = torch.zeros(c, nb, dtype=torch.uint8, device=device)
        self.dists = torch.zeros(c, nb, dtype=torch.uint8, device=device)
        self.pattern = torch.zeros(c, nb, self.nbw, dtype=torch.int64, device=device)
        self.accum = torch.zeros(c, 2, dtype=torch.int64, device=device)
        self.struct = ClusterStateStruct(n_clusters, nb, self.nbw, C.sizeof(ClusterStateStruct), self.info.data_ptr(), self.ratio.data_ptr(),
                                         self.vert.data_ptr(), self.slash.data_ptr(), self.cols.data_ptr(),
                                         self.dists.data_ptr(), self.pattern.data_ptr(), self.accum.data_ptr(),
                                         self.avg_map.data_ptr() if keep_maps else None)
        self.reset()

    def reset(self):
        """No pivot, no pattern (attention_sharing.py:41-78); enqueued on the current stream."""
        self.info.zero_()
        self.info[:, 0] = -1
        self.accum.zero_()  # (zero between completed pivot updates anyway; a reset must not depend on that)

    def ref(self):
        return C.byref(self.struct)


def share_decide(state: ClusterState, head_cluster, layer_idx, vert_blk, slash_blk, use_qa, nv, ns, min_blocks,
                 similarity_threshold, fallback_threshold):
    """-> (decision, js_v, js_s, nv_final, ns_final) (attention_sharing.py:204-301)."""
    lib = _lib.load()
    hq = vert_blk.shape[0]
    dev = vert_blk.device
    decision = torch.empty(hq, dtype=torch.int32, device=dev)
    js_v = torch.empty(hq, dtype=torch.float32, device=dev)
    js_s = torch.empty(hq, dtype=torch.float32, device=dev)
    nv_f = torch.empty(hq, dtype=torch.int32, device=dev)
    ns_f = torch.empty(hq, dtype=torch.int32, device=dev)
    st = lib.sp_share_decide(state.ref(), _ptr(head_cluster), layer_idx, hq, _ptr(vert_blk), _ptr(slash_blk),
                             _ptr(use_qa), _ptr(nv), _ptr(ns), min_blocks, similarity_threshold, fallback_threshold,
                             _ptr(decision), _ptr(js_v), _ptr(js_s), _ptr(nv_f), _ptr(ns_f), _stream(dev))
    _lib.check(st, "sp_share_decide")
    return decision, js_v, js_s, nv_f, ns_f


def build_mask(state: ClusterState, head_cluster, decision, vert_blk, slash_blk, nv_f, ns_f) -> torch.Tensor:
    """-> bit mask int64 [Hq, nb, nbw] (attention_sharing.py:303-337)."""
    lib = _lib.load()
    hq, nb = vert_blk.shape
    mask = torch.empty(hq, nb, (nb + 63) // 64, dtype=torch.int64, device=vert_blk.device)
    st = lib.sp_build_mask(state.ref(), _ptr(head_cluster), _ptr(decision), _ptr(vert_blk), _ptr(slash_blk),
                           _ptr(nv_f), _ptr(ns_f), hq, nb, _ptr(mask), _stream(vert_blk.device))
    _lib.check(st, "sp_build_mask")
    return mask


def queryaware_select(qbar, kbar, decision, mask, pattern_threshold, flags=_lib.SP_FLAG_LOGITS_BF16,
                      probs: Optional[torch.Tensor] = None) -> torch.Tensor:
    """ORs the query-aware selection into mask for heads with decision == QA; returns the probs scratch."""
    lib = _lib.load()
    nb, hq, d = qbar.shape
    hkv = kbar.shape[1]
    if probs is None:
        probs = torch.empty(hq, nb, nb, dtype=torch.float32, device=qbar.device)
    ws = _workspace("cover_select", lib.sp_cover_select_workspace_bytes(hq), qbar.device)
    st = lib.sp_queryaware_select_bf16(_ptr(qbar), _ptr(kbar), _ptr(decision), hq, hkv, d, nb, flags,
                                       pattern_threshold, _ptr(probs), _ptr(mask), _ptr(ws), ws.numel(), _stream(qbar.device))
    _lib.check(st, "sp_queryaware_select_bf16")
    return probs


def cover_select_global(x: torch.Tensor, score: float, mask: torch.Tensor, enable: Optional[torch.Tensor] = None):
    """x fp32 [V, nb, nb]; ORs the kept lower-triangular entries into mask int64 [V, nb, nbw] (attn/utils.py:53-57)."""
    lib = _lib.load()
    assert x.dtype == torch.float32 and x.is_contiguous() and mask.is_contiguous()
    v, nb, _ = x.shape
    ws = _workspace("cover_select", lib.sp_cover_select_workspace_bytes(v), x.device)
    st = lib.sp_cover_select_global(_ptr(x), _ptr(enable), v, nb, score, _ptr(mask), _ptr(ws), ws.numel(), _stream(x.device))
    _lib.check(st, "sp_cover_select_global")
    return mask


def cover_select_rows(x: torch.Tensor, thr: float) -> torch.Tensor:
    """x fp32 [nb, nb] -> pattern int64 [nb, nbw] (attn/utils.py:60-76)."""
    lib = _lib.load()
    assert x.dtype == torch.float32 and x.is_contiguous() and x.dim() == 2
    nb = x.shape[0]
    pat = torch.empty(nb, (nb + 63) // 64, dtype=torch.int64, device=x.device)
    _lib.check(lib.sp_cover_select_rows(_ptr(x), nb, thr, _ptr(pat), _stream(x.device)), "sp_cover_select_rows")
    return pat


def attention_workspace(n: int, hq: int, hkv: int, d: int, block_size: int, device, max_pivots: int = 0):
    """-> (buffer, bytes in use) of the attention call's scratch on torch's CURRENT stream: the key-major repack of V,
    the scheduler area, the pivots' row statistics and, for max_pivots > 0, room for that many heads' block sums."""
    lib = _lib.load()
    need = lib.sp_attn_workspace_bytes(n, hq, hkv, d, block_size)
    if max_pivots > 0:
        need = (need + 255) // 256 * 256 + min(max_pivots, hq) * lib.sp_attn_pivot_scratch_bytes(n, block_size)
    return _workspace("attn_vt", need, device), need


def repack_v(v: torch.Tensor, block_size: int, ws: torch.Tensor) -> None:
    """Key-major repack of v [Hkv, N, D] into the attention workspace (the step depends on v alone)."""
    lib = _lib.load()
    _check_hnd(v, "v")
    hkv, n, d = v.shape
    st = lib.sp_attn_repack_v_bf16(_ptr(v), n, hkv, d, v.stride(1), v.stride(0), block_size, _ptr(ws), ws.numel(),
                                   _stream(v.device))
    _lib.check(st, "sp_attn_repack_v_bf16")


def block_sparse_attention(q, k, v, mask, block_size, softmax_scale, decision=None, avg_attn=None, max_pivots=0,
                           workspace=None, pair_rows=False, half_channels=False):
    """q [Hq,N,D], k/v [Hkv,N,D] views, mask int64 [Hq,nb,nbw] -> out bf16 [N,Hq,D] contiguous.

    Reference: triton_block_wise_prefill_attention (shareprefill_attn.py:474-620).  avg_attn (fp32 [Hq,nb,nb],
    zero-filled) receives the block-averaged attention map of the heads whose decision is DENSE; max_pivots = how
    many such heads there can be (an upper bound the host knows): the workspace then has room to keep their block
    sums during the forward pass, which saves the second pass over Q.K^T.
    workspace: (buffer, bytes) from attention_workspace into which repack_v has ALREADY put this v (and the current
    stream has been made to wait for that); by default the call takes the buffer and repacks itself.
    pair_rows: skip the per-call analysis of which query blocks share a work item (a dense mask has no use for it).
    half_channels: q, k and v are zero beyond channel 64 (a smaller head_dim zero-padded to 128): the kernel skips
    those channels and leaves channels 64.. of out unwritten."""
    lib = _lib.load()
    _check_hnd(q, "q")
    _check_hnd(k, "k")
    _check_hnd(v, "v")
    hq, n, d = q.shape
    hkv = k.shape[0]
    assert q.shape[1] == k.shape[1] == v.shape[1], "q_len must equal k_len"
    assert mask.is_contiguous() and mask.dtype == torch.int64
    dev = q.device
    out = torch.empty(n, hq, d, dtype=torch.bfloat16, device=dev)
    if workspace is None:
        pivots = max_pivots if (avg_attn is not None and decision is not None) else 0
        ws, need = attention_workspace(n, hq, hkv, d, block_size, dev, pivots)
        repack_v(v, block_size, ws)
    else:
        ws, need = workspace
    timer = kernel_timer
    if timer is not None:
        timer.start("attn")
    st = lib.sp_block_sparse_attn_fwd_bf16(_ptr(q), _ptr(k), _ptr(v), n, hq, hkv, d, q.stride(1), q.stride(0),
                                           k.stride(1), k.stride(0), v.stride(1), v.stride(0), block_size,
                                           softmax_scale, _ptr(mask), _ptr(decision), _ptr(out), _ptr(avg_attn),
                                           _ptr(ws), need,
                                           _lib.SP_ATTN_V_REPACKED | (_lib.SP_ATTN_PAIR_ROWS if pair_rows else 0)
                                           | (_lib.SP_ATTN_HALF_CHANNELS if half_channels else 0),
                                           _stream(dev))
    if timer is not None:
        timer.stop("attn")
    _lib.check(st, "sp_block_sparse_attn_fwd_bf16")
    return out


def decode_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, softmax_scale: float,
                     out: Optional[torch.Tensor] = None, static_scratch: bool = False) -> torch.Tensor:
    """q bf16 [Hq, D] (one token), k / v bf16 [Hkv, N, D] views -> out bf16 [Hq, D].

    Reference: the flash_attn_func decode branch (shareprefill_attn.py:146-155).  static_scratch=True takes the
    entry point that allocates nothing (sp_decode_attn_static_bf16: the chunk partials live in an 8 MiB array built
    into the library instead of a torch workspace); pass `out` as well and the call touches no allocator at all."""
    lib = _lib.load()
    _check_hnd(k, "k")
    _check_hnd(v, "v")
    hq, d = q.shape
    hkv, n, _ = k.shape
    if q.dtype != torch.bfloat16 or q.stride(1) != 1:
        raise ValueError("q must be bfloat16 [Hq, D] with a contiguous head_dim axis")
    if out is None:
        out = torch.empty(hq, d, dtype=torch.bfloat16, device=q.device)
    elif out.dtype != torch.bfloat16 or tuple(out.shape) != (hq, d) or not out.is_contiguous() or out.device != q.device:
        raise ValueError(f"out must be a contiguous bfloat16 [{hq}, {d}] tensor on {q.device}")
    if static_scratch:
        st = lib.sp_decode_attn_static_bf16(_ptr(q), _ptr(k), _ptr(v), n, hq, hkv, d, q.stride(0), k.stride(1),
                                            k.stride(0), v.stride(1), v.stride(0), softmax_scale, _ptr(out),
                                            _stream(q.device))
        _lib.check(st, "sp_decode_attn_static_bf16")
        return out
    ws = _workspace("decode", lib.sp_decode_workspace_bytes(n, hq, hkv), q.device)
    st = lib.sp_decode_attn_bf16(_ptr(q), _ptr(k), _ptr(v), n, hq, hkv, d, q.stride(0), k.stride(1), k.stride(0),
                                 v.stride(1), v.stride(0), softmax_scale, _ptr(out), _ptr(ws), ws.numel(),
                                 _stream(q.device))
    _lib.check(st, "sp_decode_attn_bf16")
    return out


def rope_inplace(q: torch.Tensor, k: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> None:
    """Rotates q bf16 [Hq, N, D] and k bf16 [Hkv, N, D] (views with any token / head strides, contiguous head_dim)
    in place by the position embeddings cos / sin bf16 [N, D]:  x <- x*cos + rotate_half(x)*sin  with the roundings
    of the elementwise bf16 evaluation in Hugging Face's apply_rotary_pos_emb (bit-identical result).

    The reference leaves this step to the attention layer it patches (position embeddings: model_patch.py:121)."""
    lib = _lib.load()
    _check_hnd(q, "q")
    _check_hnd(k, "k")
    hq, n, d = q.shape
    hkv = k.shape[0]
    if k.shape[1] != n or k.shape[2] != d:
        raise ValueError(f"q {tuple(q.shape)} and k {tuple(k.shape)} must share N and D")
    for name, t in (("cos", cos), ("sin", sin)):
        if t.dtype != torch.bfloat16 or tuple(t.shape) != (n, d) or (n > 0 and t.stride(1) != 1) or t.device != q.device:
            raise ValueError(f"{name} must be bfloat16 [N, D] = [{n}, {d}] with a contiguous last axis on {q.device}")
    if n > 1 and cos.stride(0) != sin.stride(0):
        raise ValueError("cos and sin must share their row stride")
    st = lib.sp_rope_inplace_bf16(_ptr(q), _ptr(k), _ptr(cos), _ptr(sin), n, hq, hkv, d, q.stride(1), q.stride(0),
                                  k.stride(1), k.stride(0), cos.stride(0) if n > 1 else d, _stream(q.device))
    _lib.check(st, "sp_rope_inplace_bf16")


def attention_clock_mhz(n: int, hkv: int, d: int, block_size: int, device) -> float:
    """Average shader clock (MHz) seen by workgroup 0 of the last block_sparse_attention launch on this device
    (measurement aid; synchronises the current stream)."""
    import ctypes
    lib = _lib.load()
    ws = _workspaces.get(("attn_vt", str(device), _stream_handle(device)))
    if ws is None:
        raise RuntimeError("no attention launch on this device and stream yet")
    buf = (ctypes.c_int64 * 2)()
    st = lib.sp_attn_last_launch_clocks(_ptr(ws), n, hkv, d, block_size, ctypes.cast(buf, ctypes.c_void_p), _stream(device))
    _lib.check(st, "sp_attn_last_launch_clocks")
    return float(buf[0]) / (float(buf[1]) / 100.0) if buf[1] > 0 else float("nan")


def attention_pairing(n: int, hq: int, hkv: int, d: int, block_size: int, device) -> list:
    """How the last block_sparse_attention launch on this device paired query blocks into work items: one entry per
    two adjacent heads, False = two rows of a head, True = one row of both heads (test / measurement aid;
    synchronises the current stream)."""
    import ctypes
    lib = _lib.load()
    ws = _workspaces.get(("attn_vt", str(device), _stream_handle(device)))
    if ws is None:
        raise RuntimeError("no attention launch on this device and stream yet")
    buf = (ctypes.c_uint8 * ((hq + 1) // 2))()
    st = lib.sp_attn_last_launch_pairing(_ptr(ws), n, hq, hkv, d, block_size, ctypes.cast(buf, ctypes.c_void_p),
                                         _stream(device))
    _lib.check(st, "sp_attn_last_launch_pairing")
    return [bool(x) for x in buf]


def mfma_probe_tflops(random_operands, iters: int = 1500000, reps: int = 2) -> float:
    """Sustained bf16 MFMA rate of back-to-back 32x32x16 MFMAs on every CU (measurement aid).  The default runs
    about 0.2 s per repetition, long enough for the clocks to settle under the load; the last repetition counts."""
    lib = _lib.load()
    out = torch.empty(512, dtype=torch.float32, device="cuda")
    ms = 0.0
    for _ in range(reps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record(torch.cuda.current_stream())
        _lib.check(lib.sp_diag_mfma_bf16(iters, int(random_operands), _ptr(out), _stream()), "sp_diag_mfma_bf16")
        b.record(torch.cuda.current_stream())
        b.synchronize()
        ms = a.elapsed_time(b)
    return lib.sp_diag_mfma_flops(iters) / (ms * 1e-3) / 1e12


class KernelTimer:
    """Brackets kernel launches with events on the stream they are launched on (torch's current stream).
    Set ops.kernel_timer to an instance to collect; durations are read after a synchronise."""

    def __init__(self):
        self.events = {}
        self._open = {}

    def start(self, name: str):
        ev = torch.cuda.Event(enable_timing=True)
        ev.record(torch.cuda.current_stream())
        self._open[name] = ev

    def stop(self, name: str):
        ev = torch.cuda.Event(enable_timing=True)
        ev.record(torch.cuda.current_stream())
        self.events.setdefault(name, []).append((self._open.pop(name), ev))

    def durations_ms(self, name: str):
        return [a.elapsed_time(b) for a, b in self.events.get(name, [])]


kernel_timer: Optional[KernelTimer] = None


def pivot_update(state: ClusterState, head_cluster, decision, avg_attn, pattern_threshold):
    """Stores pattern / vs_ratio of this layer's pivots into the state (attention_sharing.py:94-103)."""
    lib = _lib.load()
    hq, nb, _ = avg_attn.shape
    st = lib.sp_pivot_update(state.ref(), _ptr(head_cluster), _ptr(decision), _ptr(avg_attn), hq, nb,
                             pattern_threshold, _stream(avg_attn.device))
    _lib.check(st, "sp_pivot_update")


def mask_row_pointers(mask: torch.Tensor) -> torch.Tensor:
    """CSR row pointers int32 [Hq, nb+1] of a bit mask (shareprefill_attn.py:226-269)."""
    lib = _lib.load()
    hq, nb, _ = mask.shape
    out = torch.empty(hq, nb + 1, dtype=torch.int32, device=mask.device)
    _lib.check(lib.sp_mask_row_pointers(_ptr(mask), hq, nb, _ptr(out), _stream(mask.device)), "sp_mask_row_pointers")
    return out


def _check_block_idx(idx: torch.Tensor) -> torch.Tensor:
    if idx.dim() != 2 or not idx.is_cuda:
        raise ValueError("block ids must be a GPU tensor [Hq, K]")
    if idx.dtype != torch.int64:
        idx = idx.to(torch.int64)
    if idx.shape[1] > 0 and idx.stride(1) != 1:
        idx = idx.contiguous()
    return idx


def block_idx_to_mask(idx: torch.Tensor, nb: int) -> torch.Tensor:
    """Flat block ids [Hq, K] (row * nb + col, any order, padded with values outside the grid) -> bit mask int64
    [Hq, nb, nbw]: the reference's block_idx form (shareprefill_attn.py:484-486) turned into the form the attention
    entry point takes.  Ids above the diagonal are dropped."""
    lib = _lib.load()
    idx = _check_block_idx(idx)
    hq, k = idx.shape
    mask = torch.empty(hq, nb, (nb + 63) // 64, dtype=torch.int64, device=idx.device)
    st = lib.sp_block_idx_to_mask(_ptr(idx) if k else None, idx.stride(0), k, hq, nb, _ptr(mask), _stream(idx.device))
    _lib.check(st, "sp_block_idx_to_mask")
    return mask


def block_idx_row_pointers(idx: torch.Tensor, nb: int) -> torch.Tensor:
    """Flat block ids [Hq, K] -> CSR row pointers int32 [Hq, nb+1] (count_kernel, shareprefill_attn.py:187-223)."""
    lib = _lib.load()
    idx = _check_block_idx(idx)
    hq, k = idx.shape
    out = torch.empty(hq, nb + 1, dtype=torch.int32, device=idx.device)
    st = lib.sp_block_idx_row_pointers(_ptr(idx) if k else None, idx.stride(0), k, hq, nb, _ptr(out),
                                       _stream(idx.device))
    _lib.check(st, "sp_block_idx_row_pointers")
    return out


# ---- mask format helpers (host side, synchronising; for tests and inspection) ---------------------------
def mask_to_bool(mask: torch.Tensor, nb: int) -> torch.Tensor:
    """bit mask int64 [..., nb, nbw] -> bool [..., nb, nb]."""
    shifts = torch.arange(64, device=mask.device, dtype=torch.int64)
    bits = (mask.unsqueeze(-1) >> shifts) & 1
    return bits.reshape(*mask.shape[:-1], -1)[..., :nb].bool()


def bool_to_mask(b: torch.Tensor) -> torch.Tensor:
    """bool [..., nb, nb] -> bit mask int64 [..., nb, nbw]."""
    nb = b.shape[-1]
    nbw = (nb + 63) // 64
    pad = nbw * 64 - nb
    x = torch.nn.functional.pad(b.to(torch.int64), (0, pad)).reshape(*b.shape[:-1], nbw, 64)
    lo = (x[..., :63] << torch.arange(63, device=b.device, dtype=torch.int64)).sum(-1)
    hi = torch.where(x[..., 63] != 0, torch.tensor(-(2 ** 63), dtype=torch.int64, device=b.device),
                     torch.tensor(0, dtype=torch.int64, device=b.device))
    return (lo | hi).contiguous()


def mask_to_block_idx(mask: torch.Tensor, nb: int):
    """bit mask [Hq, nb, nbw] -> list[Hq] of sorted unique flat ids (row*nb+col), the reference's block_idx."""
    b = mask_to_bool(mask, nb)
    return [torch.nonzero(b[h].reshape(-1)).reshape(-1) for h in range(b.shape[0])]

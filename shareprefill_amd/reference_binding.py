"""The binding a maintainer of the reference would add to swap only the device code (shareprefill/attn/ stays, its
Triton kernels go): a ctypes stub over the C ABI with drop-in replacements for triton_bnhd_pool (attn/utils.py:211-261)
and triton_block_wise_prefill_attention (shareprefill_attn.py:474-620).  Self-contained on purpose (it uses nothing of
this package but the built library), kept here so that it is exercised by the tests."""

import os

import ctypes as C, torch
_lib = C.CDLL(os.environ.get("SHAREPREFILL_HIP_LIB") or os.path.join(os.path.dirname(os.path.abspath(__file__)),
                                                                 "csrc", "libshareprefill_hip.so"))
_P, _I64, _I32, _F, _SZ, _U32 = C.c_void_p, C.c_int64, C.c_int32, C.c_float, C.c_size_t, C.c_uint32
_lib.sp_pool_avg_bf16.argtypes = [_P, _P, _I64, _I32, _I32, _I64, _I64, _I32, _I32, _P, _P]
_lib.sp_attn_workspace_bytes.restype = _SZ
_lib.sp_attn_workspace_bytes.argtypes = [_I64, _I32, _I32, _I32, _I32]
_lib.sp_block_sparse_attn_fwd_bf16.argtypes = [_P, _P, _P, _I64, _I32, _I32, _I32, _I64, _I64, _I64, _I64, _I64, _I64,
                                               _I32, _F, _P, _P, _P, _P, _P, _SZ, _U32, _P]
_lib.sp_block_idx_to_mask.argtypes = [_P, _I64, _I64, _I32, _I32, _P, _P]
_lib.sp_last_error.restype = C.c_char_p

def _check(rc):
    if rc: raise RuntimeError(_lib.sp_last_error().decode())

def _stream(): return C.c_void_p(torch.cuda.current_stream().cuda_stream)

def hip_bnhd_pool(x, kernel_size):                       # replaces triton_bnhd_pool (attn/utils.py:211-261)
    b, n, h, d = x.shape; assert b == 1
    y = torch.empty(1, -(-n // kernel_size), h, d, dtype=x.dtype, device=x.device)
    _check(_lib.sp_pool_avg_bf16(x.data_ptr(), y.data_ptr(), n, h, d, x.stride(1), x.stride(2), kernel_size, 0,
                                 None, _stream()))
    return y

def ids_to_mask(block_idx, nb):                           # reference id lists -> bit mask [H, nb, ceil(nb/64)]
    ids = torch.nn.utils.rnn.pad_sequence([t.reshape(-1).long() for t in block_idx[0]], batch_first=True,
                                          padding_value=nb * (nb + 1))   # the reference's own padding value
    h, k = ids.shape
    mask = torch.empty(h, nb, (nb + 63) // 64, dtype=torch.int64, device=ids.device)
    _check(_lib.sp_block_idx_to_mask(ids.data_ptr(), ids.stride(0), k, h, nb, mask.data_ptr(), _stream()))
    return mask

def hip_block_wise_prefill_attention(q, k, v, block_idx, use_dense, block_size, softmax_scale):
    # replaces triton_block_wise_prefill_attention (shareprefill_attn.py:474-620); q [1,N,Hq,D], k/v [1,N,Hkv,D]
    # (pass the UN-expanded k, v: skip _maybe_repeat_kv, shareprefill_attn.py:99-104)
    _, n, hq, d = q.shape; hkv = k.shape[2]; nb = -(-n // block_size)
    mask = ids_to_mask(block_idx, nb)
    decision = use_dense[0].to(torch.int32)               # 1 = SP_DEC_DENSE
    out = torch.empty_like(q)
    avg = torch.zeros(1, hq, nb, nb, dtype=torch.float32, device=q.device)
    ws = torch.empty(_lib.sp_attn_workspace_bytes(n, hq, hkv, d, block_size), dtype=torch.uint8, device=q.device)
    _check(_lib.sp_block_sparse_attn_fwd_bf16(
        q.data_ptr(), k.data_ptr(), v.data_ptr(), n, hq, hkv, d, q.stride(1), q.stride(2), k.stride(1), k.stride(2),
        v.stride(1), v.stride(2), block_size, softmax_scale, mask.data_ptr(), decision.data_ptr(), out.data_ptr(),
        avg.data_ptr(), ws.data_ptr(), ws.numel(), 0, _stream()))
    return out, avg

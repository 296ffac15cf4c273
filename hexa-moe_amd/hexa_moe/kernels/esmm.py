"""`ESMM` with the Triton sibling's argument list (reference: hexa_moe_triton/hexa_moe/kernels/esmm.py:249-295)."""
import torch

from .. import _lib, ops
from .basics import route_of_lists


def ESMM(toks, w, b, tok_ids_list, exp_ids_list):
    """c[t] = toks[t] @ w[e(t)] + b[e(t)] for every token named in the lists, zeros for the others.

    toks [num_toks, in]; w [num_exps, in, out]; b [num_exps, out] or an empty tensor; tok_ids_list int32
    [P] 1-based token ids (0 = padding); exp_ids_list int32 [P // 16].  Returns c [num_toks, out] in toks' type."""
    assert toks.is_contiguous() and w.is_contiguous() and toks.shape[1] == w.shape[1], "Matrix A must be contiguous"
    num_toks = toks.shape[0]
    num_exps, _, num_out_dims = w.shape
    route = route_of_lists(tok_ids_list, exp_ids_list, num_toks, num_exps)
    bias = None
    if b is not None and b.numel():
        assert num_out_dims == b.shape[1] and num_exps == b.shape[0]
        bias = b.contiguous()
        if bias.dtype not in (toks.dtype, torch.float32):
            bias = bias.to(torch.float32)                     # the reference promotes the bias to fp32 as well
    c = torch.zeros(1, num_toks, num_out_dims, dtype=toks.dtype, device=toks.device)
    wk = w if w.dtype in (toks.dtype, torch.float32) else w.to(toks.dtype)
    ops.esmm(toks, wk, bias, route, False, _lib.HEXA_W_IN_OUT, out=c, accumulate=True)
    return c[0]

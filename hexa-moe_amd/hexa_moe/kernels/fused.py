"""`es_fused` with the Triton sibling's argument list (reference:
hexa_moe_triton/hexa_moe/kernels/fused.py:382-450: ESS, ESMM and ESTMM of one backward step from one launch)."""
import torch

from .. import _lib, ops
from .basics import route_of_lists


def es_fused(tok1, tok2, w, tok_ids_list, exp_ids_list, exp_start_list, num_exps, bias=True):
    """tok1 [num_toks, out] (the incoming gradient), tok2 [num_toks, in] (the forward's input), w [num_exps, out, in];
    lists as for ESMM; exp_start_list int32 [num_exps + 1] (kept for the signature: the library rebuilds the
    segment starts from the lists).  Returns ([r_ess,] r_esmm, r_estmm):
      r_ess   [num_exps, out]      per-expert sums of tok1's rows                    (only with bias=True)
      r_esmm  [num_toks, in]       tok1[t] @ w[e(t)]   (rows of tokens not in the lists are zero; the reference
                                   leaves them uninitialised)
      r_estmm [num_exps, out, in]  per-expert tok1^T @ tok2
    r_esmm has tok1's type, r_ess and r_estmm have w's."""
    assert tok1.dtype == tok2.dtype
    assert tok1.shape[0] == tok2.shape[0]
    assert tok2.shape[1] == w.shape[2] and num_exps == w.shape[0] and tok1.shape[1] == w.shape[1]
    assert exp_start_list.shape[0] == 1 + num_exps
    assert tok1.is_contiguous() and tok2.is_contiguous()
    num_toks, num_out_dims = tok1.shape
    num_in_dims = tok2.shape[1]
    route = route_of_lists(tok_ids_list, exp_ids_list, num_toks, num_exps)
    wk = w.contiguous()
    if wk.dtype not in (tok1.dtype, torch.float32):
        wk = wk.to(tok1.dtype)
    # ESMM task: r_esmm = tok1 . w[e] with w [E][out][in] read as an [E][in'=out][out'=in] weight
    r_esmm = torch.zeros(1, num_toks, num_in_dims, dtype=tok1.dtype, device=tok1.device)
    ops.esmm(tok1, wk, None, route, False, _lib.HEXA_W_IN_OUT, out=r_esmm, accumulate=True)
    grad_dt = torch.float32 if w.dtype == torch.float32 else tok1.dtype
    r_estmm = ops.estmm(tok1, tok2, route, False, False, out_dtype=grad_dt).to(w.dtype)
    if bias:
        r_ess = ops.ess(tok1, route, False, out_dtype=grad_dt).to(w.dtype)
        return r_ess, r_esmm[0], r_estmm
    return r_esmm[0], r_estmm

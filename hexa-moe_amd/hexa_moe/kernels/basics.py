"""`counter`: per-expert token lists in the Triton sibling's format (reference:
hexa_moe_triton/hexa_moe/kernels/basics.py:89-118 -- token_count_kernel, padding_kernel, assign_tok_kernel,
assign_exp_kernel and the host loop between them)."""
import torch

from .. import _lib, ops
from . import constant


def counter(routing, num_exps):
    """routing: [T] expert choice of one routing slot (int32 / int64, on the GPU).

    Returns (num_expanded_toks, exp_start_list, tok_ids_list, exp_ids_list) as the reference does:
      num_expanded_toks  Python int: sum over experts of their token counts rounded up to multiples of 16
      exp_start_list     int32 [num_exps + 1]: exclusive prefix of the rounded counts
      tok_ids_list       int32 [num_expanded_toks]: 0-based token ids grouped by expert, -1 in the padding
                         (the reference's callers add 1 before handing it to ESMM / es_fused)
      exp_ids_list       int32 [num_expanded_toks // 16]: the expert of every chunk of 16 list positions
    Within an expert the ids ascend (the reference's order depends on the timing of its atomics).  Ids outside
    [0, num_exps) are skipped, as there.  One read of a device scalar (the list length), where the reference
    reads num_exps of them."""
    ops._dev(routing)
    if routing.dim() != 1:
        raise ValueError("counter: routing must be one slot's [T] expert ids")
    r = routing.to(torch.int32).contiguous()
    T, E = r.shape[0], int(num_exps)
    dev = r.device
    lib = _lib.load()
    counts = torch.empty(E, dtype=torch.int32, device=dev)
    exp_start_list = torch.empty(E + 1, dtype=torch.int32, device=dev)
    units = max(1, (T + _lib.HEXA_ROUTE_UNIT - 1) // _lib.HEXA_ROUTE_UNIT)
    scratch = torch.empty(units * E, dtype=torch.int32, device=dev)
    st = ops._stream()
    _lib.check(lib.hexa_token_count(counts.data_ptr(), exp_start_list.data_ptr(), r.data_ptr(), T, E,
                                    constant.MAX_TOKEN_CHUNK, scratch.data_ptr(), st), "hexa_token_count")
    num_expanded_toks = int(exp_start_list[E].item())
    tok_ids_list = torch.full((num_expanded_toks,), -1, dtype=torch.int32, device=dev)
    per_pos = torch.full((num_expanded_toks,), -1, dtype=torch.int32, device=dev)
    _lib.check(lib.hexa_token_assign(tok_ids_list.data_ptr(), per_pos.data_ptr(), exp_start_list.data_ptr(), r.data_ptr(),
                                     T, E, scratch.data_ptr(), st), "hexa_token_assign")
    chunks = (exp_start_list[1:] - exp_start_list[:-1]) // constant.MAX_TOKEN_CHUNK
    exp_ids_list = torch.repeat_interleave(torch.arange(E, dtype=torch.int32, device=dev), chunks.long())
    return num_expanded_toks, exp_start_list, tok_ids_list, exp_ids_list


def route_of_lists(tok_ids_list, exp_ids_list, num_toks, num_exps):
    """Routing metadata of the HIP operators from one slot's lists in the operators' format: 1-based token
    ids (0 = padding) and one expert id per chunk of 16 positions."""
    ops._dev(tok_ids_list, exp_ids_list)
    if tok_ids_list.dtype != torch.int32 or exp_ids_list.dtype != torch.int32:
        raise TypeError("tok_ids_list and exp_ids_list must be int32")
    if tok_ids_list.shape[0] != constant.MAX_TOKEN_CHUNK * exp_ids_list.shape[0]:
        raise ValueError("tok_ids_list must hold 16 positions per entry of exp_ids_list")
    tok0 = (tok_ids_list - 1).contiguous()                      # 0-based, padding -> -1 (dropped by the library)
    per_pos = exp_ids_list.repeat_interleave(constant.MAX_TOKEN_CHUNK).contiguous()
    ends = torch.tensor([0, tok0.shape[0]], dtype=torch.int32, device=tok0.device)
    return ops.route_from_padded_lists(tok0, per_pos, ends, int(num_toks), 1, int(num_exps))

"""The reference extension's five operators, same names and argument lists, on the HIP library.

Mirrors the pybind module `hexa_moe_cuda` of the reference (hexa_moe_cuda/hexa_moe/torch/
hexa_moe_ops.cpp:277-301): TOKEN_COUNT, TOKEN_ASSIGN, ESMM_TENSOR_CORE, FUSED_GRAD,
FUSED_GRAD_NO_BIAS.  All results are written in place into caller-allocated tensors; the matmul
results are accumulated (+=) as in the reference, whose callers zero them first
(impls/layers.py:230-231, 404-405, 432-436).

Differences that a caller can observe:
  * segments are not padded: expanded_tokens_per_expert is the exact exclusive prefix, so the lists
    the caller sizes from its last entry (impls/layers.py:238) have exactly num_tokens entries.
    set_pad(16) switches TOKEN_COUNT / TOKEN_ASSIGN to the reference's 16-padded format; the matmul
    ops take either format (padded lists are compacted on the device from num_expanded_tokens, the
    cumulative list lengths, before the operators run).
  * the order inside a segment is ascending token id (the reference's depends on atomics).
  * element types come from the tensors; the *_dtype_full flags are checked against them.  bf16 is
    accepted wherever fp16 is.
  * unsupported combinations raise instead of printing and returning.
"""
import torch

from hexa_moe import _lib, ops

_pad = 1


def set_pad(pad):
    """Segment granularity of TOKEN_COUNT / TOKEN_ASSIGN (1 = unpadded, 16 = the reference's)."""
    global _pad
    if int(pad) < 1:
        raise ValueError("pad must be >= 1")
    _pad = int(pad)


def _scratch(num_tokens, num_routings, device):
    units = max(1, -(-int(num_tokens) // _lib.HEXA_ROUTE_UNIT))
    return torch.empty(units * int(num_routings), dtype=torch.int32, device=device)


def _i32(t, what):
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise TypeError(f"{what} must be a contiguous int32 tensor")
    ops._dev(t)
    return t


def _forget_routes_of(*written):
    """Drop the cached routing metadata of every list tensor this call is about to rewrite.  The operators below write
    through raw device pointers, which does not advance a tensor's version counter, so the cache key alone would not
    notice a second TOKEN_ASSIGN into the same preallocated lists."""
    spans = [(t.data_ptr(), t.data_ptr() + t.numel() * t.element_size()) for t in written if t is not None]
    for key, (_, tok, exp, cum) in list(_route_cache.items()):
        for held in (tok, exp, cum):
            if held is None:
                continue
            lo, hi = held.data_ptr(), held.data_ptr() + held.numel() * held.element_size()
            if any(lo < b and a < hi for a, b in spans):
                del _route_cache[key]
                break


def TOKEN_COUNT(tokens_per_expert, expanded_tokens_per_expert, routings, num_tokens, num_routings):
    _i32(tokens_per_expert, "tokens_per_expert"); _i32(expanded_tokens_per_expert, "expanded_tokens_per_expert")
    _i32(routings, "routings")
    _forget_routes_of(tokens_per_expert, expanded_tokens_per_expert)
    assert tokens_per_expert.numel() >= num_routings and expanded_tokens_per_expert.numel() >= num_routings + 1
    assert routings.numel() >= num_tokens
    scratch = _scratch(num_tokens, num_routings, routings.device)
    rc = _lib.load().hexa_token_count(tokens_per_expert.data_ptr(), expanded_tokens_per_expert.data_ptr(),
                                      routings.data_ptr(), int(num_tokens), int(num_routings), _pad,
                                      scratch.data_ptr(), ops._stream())
    _lib.check(rc, "TOKEN_COUNT")


def TOKEN_ASSIGN(token_idx_list, expert_idx_list, expanded_tokens_per_expert, routings, num_tokens, num_routings):
    _i32(token_idx_list, "token_idx_list"); _i32(expert_idx_list, "expert_idx_list")
    _i32(expanded_tokens_per_expert, "expanded_tokens_per_expert"); _i32(routings, "routings")
    _forget_routes_of(token_idx_list, expert_idx_list)
    scratch = _scratch(num_tokens, num_routings, routings.device)
    rc = _lib.load().hexa_token_assign(token_idx_list.data_ptr(), expert_idx_list.data_ptr(),
                                       expanded_tokens_per_expert.data_ptr(), routings.data_ptr(), int(num_tokens),
                                       int(num_routings), scratch.data_ptr(), ops._stream())
    _lib.check(rc, "TOKEN_ASSIGN")


_route_cache = {}          # (list pointers, versions, sizes) -> Route; a handful of entries (one per live routing)
_ROUTE_CACHE_MAX = 16


def _route(token_idx_list, expert_idx_list, num_expanded_tokens, num_tokens, top_k, num_routings):
    """Routing metadata of the operators for the caller's lists.  The reference's layer calls the matmul ops several
    times per step with the same lists (impls/layers.py:256-274, 409-451); the metadata (and the ESTMM work plan
    that hangs off it) is built once per list contents: the cache key holds the tensors' addresses and version
    counters, so lists that were rewritten in place by torch are rebuilt, and TOKEN_COUNT / TOKEN_ASSIGN drop the
    entries of the tensors they write (_forget_routes_of)."""
    _i32(token_idx_list, "token_idx_list"); _i32(expert_idx_list, "expert_idx_list")
    if token_idx_list.numel() != expert_idx_list.numel():
        raise ValueError("token_idx_list and expert_idx_list differ in length")
    key = (token_idx_list.data_ptr(), token_idx_list._version, expert_idx_list.data_ptr(), expert_idx_list._version,
           token_idx_list.numel(), int(num_tokens), int(top_k), int(num_routings),
           None if num_expanded_tokens is None else (num_expanded_tokens.data_ptr(), num_expanded_tokens._version))
    hit = _route_cache.get(key)
    if hit is not None:
        return hit[0]
    if token_idx_list.numel() == num_tokens * top_k:     # exact lists: nothing to drop
        route = ops.route_from_lists(token_idx_list, expert_idx_list, int(num_tokens), int(top_k), int(num_routings))
    elif token_idx_list.numel() < num_tokens * top_k:
        raise ValueError("the lists hold fewer than top_k * num_tokens entries")
    else:
        _i32(num_expanded_tokens, "num_expanded_tokens")
        route = ops.route_from_padded_lists(token_idx_list, expert_idx_list, num_expanded_tokens, int(num_tokens),
                                            int(top_k), int(num_routings))
    if len(_route_cache) >= _ROUTE_CACHE_MAX:
        _route_cache.pop(next(iter(_route_cache)))
    # the entry keeps the list tensors alive, so their addresses cannot be reused by other lists while it exists
    _route_cache[key] = (route, token_idx_list, expert_idx_list, num_expanded_tokens)
    return route


def clear_route_cache():
    _route_cache.clear()


def _check_flag(t, full, what):
    if (t.dtype == torch.float32) != bool(full):
        raise TypeError(f"{what}: dtype flag does not match the tensor ({t.dtype})")


def ESMM_TENSOR_CORE(result, tokens, weights, bias, token_idx_list, expert_idx_list, num_expanded_tokens,
                     x_dtype_full, w_dtype_full, b_dtype_full, m2s, num_tokens, top_k, num_in_dims, num_out_dims,
                     num_routings):
    T, k, E = int(num_tokens), int(top_k), int(num_routings)
    _check_flag(tokens, x_dtype_full, "tokens"); _check_flag(weights, w_dtype_full, "weights")
    route = _route(token_idx_list, expert_idx_list, num_expanded_tokens, T, k, E)
    x = tokens.reshape((k, T, num_in_dims) if m2s else (T, num_in_dims))
    w = weights.reshape(E, num_in_dims, num_out_dims)
    b = bias.reshape(E, num_out_dims) if bias is not None and bias.numel() > 0 else None
    out = result.reshape((T, num_out_dims) if m2s else (k, T, num_out_dims))
    assert out.data_ptr() == result.data_ptr(), "result must be contiguous"
    ops.esmm(x, w, b, route, bool(m2s), _lib.HEXA_W_IN_OUT, out=out, accumulate=True)


def _fused(j_b, j_x, j_w, j_y, w, x, token_idx_list, expert_idx_list, num_expanded_tokens, m2s, num_tokens, top_k,
           num_in_dims, num_out_dims, num_routings):
    T, k, E = int(num_tokens), int(top_k), int(num_routings)
    route = _route(token_idx_list, expert_idx_list, num_expanded_tokens, T, k, E)
    for t in (j_x, j_w, j_y, w, x) + ((j_b,) if j_b is not None else ()):
        ops._dev(t)
        if not t.is_contiguous():
            raise TypeError("FUSED_GRAD: tensors must be contiguous")
    ws = torch.empty((k - 1) * T * int(num_in_dims), dtype=j_x.dtype, device=j_x.device) if (m2s and k > 1) else None
    # balanced ESTMM and split ESS walk, as the layer's own calls get them (ops.estmm / ops.ess)
    plan = scratch = ess_ws = None
    slots = 0
    mn = int(num_out_dims) * int(num_in_dims)
    if j_y.dtype != torch.float32:
        if T * k >= 128 * E and mn % 4 == 0:
            slots = min(2 * E, (256 << 20) // (mn * 4))
            slots = slots if slots >= 2 else 0
        plan = route.estmm_plan(slots, int(num_out_dims), int(num_in_dims))
        if slots:
            scratch = torch.empty(slots * mn, dtype=torch.float32, device=j_y.device)
    if j_b is not None and T * k >= 256 * E:
        ess_ws = torch.empty(8 * E * int(num_out_dims), dtype=torch.float32, device=j_y.device)
    rc = _lib.load().hexa_fused_grad(
        j_b.data_ptr() if j_b is not None else None, j_x.data_ptr(), j_w.data_ptr(), j_y.data_ptr(), w.data_ptr(),
        x.data_ptr(), route.blob.data_ptr(), int(bool(m2s)), 1, T, k, int(num_in_dims), int(num_out_dims), E,
        ops._dt(j_y), ops._dt(w), ops._dt(j_x), ops._dt(j_w), ops._dt(j_b) if j_b is not None else 0,
        ws.data_ptr() if ws is not None else None, plan.data_ptr() if plan is not None else None, slots,
        scratch.data_ptr() if scratch is not None else None, ess_ws.data_ptr() if ess_ws is not None else None,
        ess_ws.numel() if ess_ws is not None else 0, ops._stream())
    _lib.check(rc, "FUSED_GRAD")


def FUSED_GRAD(j_b, j_x, j_w, j_y, w, x, token_idx_list, expert_idx_list, num_expanded_tokens, x_dtype_full,
               w_dtype_full, m2s, num_tokens, top_k, num_in_dims, num_out_dims, num_routings):
    _check_flag(j_y, x_dtype_full, "j_y"); _check_flag(w, w_dtype_full, "w")
    _fused(j_b, j_x, j_w, j_y, w, x, token_idx_list, expert_idx_list, num_expanded_tokens, m2s, num_tokens, top_k,
           num_in_dims, num_out_dims, num_routings)


def FUSED_GRAD_NO_BIAS(j_x, j_w, j_y, w, x, token_idx_list, expert_idx_list, num_expanded_tokens, x_dtype_full,
                       w_dtype_full, m2s, num_tokens, top_k, num_in_dims, num_out_dims, num_routings):
    _check_flag(j_y, x_dtype_full, "j_y"); _check_flag(w, w_dtype_full, "w")
    _fused(None, j_x, j_w, j_y, w, x, token_idx_list, expert_idx_list, num_expanded_tokens, m2s, num_tokens, top_k,
           num_in_dims, num_out_dims, num_routings)

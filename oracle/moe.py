"""Routing, token->expert alignment and the fused-MoE sequence on the CPU.

Test infrastructure only.

* ``topk_softmax`` (csrc/src/topk_softmax.cpp:27-34; in-tree twin
  vllm_gcu/models/deepseek_moe_quant/deepseek_moe_quant.py:168-173).
* ``grouped_topk`` (vllm_gcu/kernels/fused_moe.py:234-267 ->
  csrc/src/fused_grouped_topk.cpp:22-44; two overloads, with and without
  ``e_score_correction_bias``).
* ``moe_align_block_size`` (fused_moe.py:40-108; sizes and the pad sentinel
  ``numel`` per tests/kernels/test_moe_align.py:12-21).
* ``silu_and_mul`` (csrc/src/silu_and_mul.cpp:29-36), ``moe_sum``
  (csrc/src/moe_sum.cpp:64-80).
* ``fused_moe_gemm``: the "non-gather" grouped GEMM contract
  (csrc/src/native_vllm.h:236-255, fused_moe_quant_kernel.cpp:68-76).
* ``fused_experts``: the sequence of modular_experts.py:81-288.
"""
import numpy as np


def softmax_f32(logits: np.ndarray) -> np.ndarray:
    x = logits.astype(np.float32)
    m = x.max(axis=-1, keepdims=True)
    e = np.exp((x - m).astype(np.float32)).astype(np.float32)
    return (e / e.sum(axis=-1, keepdims=True, dtype=np.float32)).astype(np.float32)


def _stable_topk(scores: np.ndarray, k: int):
    """Descending values, ties to the lower index (the stable top-k the
    reference's CPU twin names, csrc/src/native_vllm.h:290-293)."""
    order = np.argsort(-scores, axis=-1, kind="stable")[..., :k]
    return np.take_along_axis(scores, order, axis=-1), order.astype(np.int32)


def topk_softmax(gating: np.ndarray, topk: int, renormalize: bool = False):
    """-> (weights f32 [M, T] descending, ids i32 [M, T],
    token_expert_indices i32 [M, T] with value ``k * M + row``)."""
    p = softmax_f32(gating)
    w, ids = _stable_topk(p, topk)
    M = gating.shape[0]
    tei = (np.arange(topk, dtype=np.int32)[None, :] * M +
           np.arange(M, dtype=np.int32)[:, None]).astype(np.int32)
    if renormalize:
        w = (w / w.sum(axis=-1, keepdims=True, dtype=np.float32)).astype(np.float32)
    return w.astype(np.float32), ids, tei


def grouped_topk(gating: np.ndarray, topk: int, renormalize: bool,
                 num_expert_group: int, topk_group: int,
                 scoring_func: str = "softmax", bias=None):
    """Grouped top-k routing.

    scores = softmax | sigmoid (float32).  Without bias the group score is the
    max of the group's scores; with bias the selection scores are ``scores +
    bias`` and the group score is the sum of the group's two largest selection
    scores.  The ``topk_group`` best groups are kept (ties to the lower group),
    the ``topk`` best selection scores among kept groups are taken
    (descending, ties to the lower expert), weights are gathered from the
    *un-biased* scores and optionally renormalised.
    """
    g = gating.astype(np.float32)
    if scoring_func == "softmax":
        scores = softmax_f32(g)
    elif scoring_func == "sigmoid":
        scores = (np.float32(1) / (np.float32(1) + np.exp(-g).astype(np.float32))).astype(np.float32)
    else:
        raise ValueError(scoring_func)
    M, E = scores.shape
    per = E // num_expert_group
    sel = scores if bias is None else (scores + bias.astype(np.float32)[None, :]).astype(np.float32)
    grp = sel.reshape(M, num_expert_group, per)
    if bias is None:
        gscore = grp.max(axis=-1)
    else:
        top2, _ = _stable_topk(grp, 2)
        gscore = (top2[..., 0] + top2[..., 1]).astype(np.float32)
    _, gidx = _stable_topk(gscore, topk_group)
    mask = np.zeros((M, num_expert_group), dtype=bool)
    np.put_along_axis(mask, gidx.astype(np.int64), True, axis=-1)
    emask = np.repeat(mask, per, axis=1)
    masked = np.where(emask, sel, -np.inf).astype(np.float32)
    _, ids = _stable_topk(masked, topk)
    w = np.take_along_axis(scores, ids.astype(np.int64), axis=-1).astype(np.float32)
    if renormalize:
        w = (w / w.sum(axis=-1, keepdims=True, dtype=np.float32)).astype(np.float32)
    return w, ids


def moe_align_block_size(topk_ids: np.ndarray, num_experts: int, block_size: int,
                         valid_rows=None, expert_map=None):
    """Counting sort of flat (token, slot) ids by expert, each expert's run
    padded to a multiple of ``block_size``.

    Returns ``(sorted_token_ids i32 [numel + E*(B-1)], expert_ids i32
    [len // B], num_tokens_post_pad i32 [1])``.  Entries of
    ``sorted_token_ids`` index the flattened ``topk_ids``; pads and the unused
    tail hold the sentinel ``numel``; within an expert flat ids ascend
    (stable).  ``expert_ids`` past the used blocks are left at -1 here and are
    not part of the contract.  ``valid_rows``: only the first that many rows of
    ``topk_ids`` are sorted (the ``_pad`` variant,
    csrc/src/moe_align_block_size_pad.cpp:43-47).  ``expert_map`` is applied to
    ``expert_ids`` afterwards (fused_moe.py:70-71, 106-107).
    """
    flat = topk_ids.reshape(-1).astype(np.int64)
    numel = flat.size
    top = topk_ids.shape[-1] if topk_ids.ndim > 1 else 1
    nvalid = numel if valid_rows is None else int(valid_rows) * top
    cap = numel + num_experts * (block_size - 1)
    sorted_ids = np.full(cap, numel, dtype=np.int32)
    expert_ids = np.full(cap // block_size, -1, dtype=np.int32)
    pos = 0
    for e in range(num_experts):
        idx = np.nonzero(flat[:nvalid] == e)[0]
        if idx.size == 0:
            continue
        sorted_ids[pos:pos + idx.size] = idx
        padded = -(-idx.size // block_size) * block_size
        expert_ids[pos // block_size:(pos + padded) // block_size] = e
        pos += padded
    if expert_map is not None:
        used = pos // block_size
        expert_ids[:used] = np.asarray(expert_map)[expert_ids[:used]]
    return sorted_ids, expert_ids, np.array([pos], dtype=np.int32)


def silu_and_mul(x: np.ndarray) -> np.ndarray:
    """``left * sigmoid(left) * right`` in float32 (silu_and_mul.cpp:29-36)."""
    d = x.shape[-1] // 2
    a = x[..., :d].astype(np.float32)
    b = x[..., d:].astype(np.float32)
    return (a * (np.float32(1) / (np.float32(1) + np.exp(-a).astype(np.float32))) * b).astype(np.float32)


def moe_sum(x: np.ndarray) -> np.ndarray:
    """Sum over the top-k axis (dim 1) in float32 (moe_sum.cpp:64-80)."""
    return x.astype(np.float32).sum(axis=1, dtype=np.float32)


def fused_moe_gemm(a_rows: np.ndarray, expert_weight_fn, topk_ids: np.ndarray,
                   topk: int, topk_weights=None, mul_routed_weight=False) -> np.ndarray:
    """Non-gather grouped GEMM: for every flat id t, ``C[t] = A[t // topk] @
    W[expert(t)]`` (times ``topk_weights.flat[t]`` when asked).

    ``a_rows`` float32 [M_a, K]; ``expert_weight_fn(e)`` returns the dense
    float32 ``[K, N]`` weight of expert e.  Result float32 [numel, N].
    """
    import torch
    flat = topk_ids.reshape(-1)
    out = None
    for e in np.unique(flat):
        w = torch.from_numpy(np.ascontiguousarray(expert_weight_fn(int(e))))
        rows = np.nonzero(flat == e)[0]
        a = torch.from_numpy(np.ascontiguousarray(a_rows[rows // topk]))
        c = torch.matmul(a, w).numpy()
        if out is None:
            out = np.zeros((flat.size, c.shape[1]), dtype=np.float32)
        out[rows] = c
    if mul_routed_weight:
        out = out * topk_weights.reshape(-1, 1).astype(np.float32)
    return out


def fused_experts(x, w1_fn, w2_fn, topk_weights, topk_ids, act_dtype,
                  quant_a2=None, return_slots=False):
    """modular_experts.py:81-288 on the CPU: GEMM1 -> cast -> silu_and_mul ->
    cast -> GEMM2 (routed weights applied) -> cast -> sum over slots.

    ``act_dtype``: a function rounding a float32 array to the activation dtype
    and back (the intermediate caches are stored in that dtype).
    ``quant_a2``: optional function mapping the float32 activation of GEMM2 to
    its dequantised float32 (per-token-group fp8 / int8 paths).
    """
    M, T = topk_ids.shape
    c1 = act_dtype(fused_moe_gemm(x.astype(np.float32), w1_fn, topk_ids, T))
    c2 = act_dtype(silu_and_mul(c1))
    if quant_a2 is not None:
        c2 = quant_a2(c2)
    c3 = fused_moe_gemm(c2, w2_fn, topk_ids, 1, topk_weights, True)
    c3 = act_dtype(c3).reshape(M, T, -1)
    if return_slots:                       # also the rounded per-slot terms [M, T, K] that are summed
        return act_dtype(moe_sum(c3)), c3
    return act_dtype(moe_sum(c3))

"""Sequence-mixer ops: layer norm over an fp32 residual stream, sliding-window
attention over a compressed latent cache, gated linear attention; sandwich
RMS norm with depth-weighted averaging, row-cache attention (differential /
pooled sliding window / sigmoid-weighted with an output gate) and xIELU;
post-norm residual step, minGRU scan and the clamped gated linear unit;
grouped RMS norm over a parallel residual, hashed pair embedding, squared relu
and the rotation of head rows by position.

GPU tensors go to the hand-written gfx950 kernels of the in-tree extension
``parallax_amd.ops._mix`` (bf16 or float32 activations; scores, norms, decays
and recurrent state always fp32). There is no eager fallback on a GPU: a
missing extension raises. CPU tensors run the eager torch versions in
``reference.py`` (CPU engine, tests)."""

from __future__ import annotations

from typing import Optional

import torch

from . import reference as ref

_MIX = None
_MIX_ERR: Optional[str] = None


def _mix_ext():
    global _MIX, _MIX_ERR
    if _MIX is None and _MIX_ERR is None:
        try:
            from . import _mix  # built in-tree (setup.py, PARALLAX_EXT=_mix)

            _MIX = _mix
        except ImportError as e:
            _MIX_ERR = str(e)
    if _MIX is None:
        raise RuntimeError(
            "the parallax_amd.ops._mix HIP extension is required on a GPU but "
            f"is not built (import error: {_MIX_ERR}); build it with "
            "`PARALLAX_EXT=_mix python setup.py build_ext --inplace`"
        )
    return _MIX


def has_mix_extension() -> bool:
    try:
        _mix_ext()
        return True
    except RuntimeError:
        return False


def _empty(like: torch.Tensor, dtype=None) -> torch.Tensor:
    return like.new_empty(0, dtype=dtype or like.dtype)


def add_layernorm(resid, y, scale, mult, weight, bias, eps, out_dtype):
    """resid [T, W] fp32 <- resid + mult * scale * y (in place; y None = no
    update), then layer norm with weight and bias -> [T, W] of out_dtype
    (weight None = no norm, returns None)."""
    if not resid.is_cuda:
        return ref.add_layernorm(resid, y, scale, mult, weight, bias, eps, out_dtype)
    ext = _mix_ext()
    out = torch.empty(resid.shape, dtype=out_dtype, device=resid.device) \
        if weight is not None else _empty(resid)
    ext.add_layernorm(
        resid, y if y is not None else _empty(resid),
        scale if y is not None else _empty(resid), float(mult),
        weight if weight is not None else _empty(resid),
        bias if weight is not None else _empty(resid), float(eps), out,
    )
    return out if weight is not None else None


def latent_kv_store(dkv, norm_w, eps, freq, mult, rot_dims, positions,
                    slot_mapping, cache, rank):
    """RMS-norm the first `rank` columns of dkv, rotate the rest by position,
    scatter both as one cache row per token (slot -1 = skip)."""
    if not dkv.is_cuda:
        return ref.latent_kv_store(dkv, norm_w, eps, freq, mult, rot_dims,
                                   positions, slot_mapping, cache, rank)
    _mix_ext().latent_kv_store(dkv, norm_w, float(eps), freq, float(mult),
                               int(rot_dims), positions, slot_mapping, cache,
                               int(rank))


def rope_rows(q, col0, rot_w, freq, mult, rot_dims, positions):
    """q [T, H, D]: columns [col0, col0+rot_w) of every head, rotated on their
    first rot_dims dimensions, as a new fp32 [T, H, rot_w]."""
    if not q.is_cuda:
        return ref.rope_rows(q, col0, rot_w, freq, mult, rot_dims, positions)
    out = torch.empty(q.shape[0], q.shape[1], rot_w, dtype=torch.float32,
                      device=q.device)
    _mix_ext().rope_rows(out, q, int(col0), freq, float(mult), int(rot_dims),
                         positions)
    return out


def latent_window_attention(q_lat, q_rot, cache, block_tables, token_seq,
                            positions, window, scale, max_seq_len=0):
    """Softmax attention of absorbed queries over the paged latent cache with
    a sliding window: token at position p sees keys p-window+1 .. p of its
    sequence. q_lat [T, H, rank] fp32, q_rot [T, H, rot_w] fp32, token_seq [T]
    int32 (None: token i is sequence i). max_seq_len: the longest context in
    the batch as the host knows it (0 = the block tables' capacity); it only
    sizes the split of long windows over workgroups. Returns fp32 [T, H, rank]."""
    if not q_lat.is_cuda:
        return ref.latent_window_attention(q_lat, q_rot, cache, block_tables,
                                           token_seq, positions, window, scale)
    out = torch.empty_like(q_lat)
    _mix_ext().latent_window_attention(
        out, q_lat, q_rot, cache, block_tables,
        token_seq if token_seq is not None
        else _empty(positions), positions, int(window), float(scale),
        int(max_seq_len) or block_tables.shape[1] * cache.shape[1],
    )
    return out


def gla_recurrence(q, k, v, z, z_bias, state, slots, cu, positions, inv_tau,
                   q_scale):
    """Gated-linear-attention recurrence over packed sequences; the fp32
    state [slots, H, dk, dv] is read (or started from zero at position 0) and
    written back. cu [B+1] int32 token bounds (None: one token each). Returns
    fp32 o [T, H, dv]."""
    if not q.is_cuda:
        return ref.gla_recurrence(q, k, v, z, z_bias, state, slots, cu,
                                  positions, inv_tau, q_scale)
    H, dv = state.shape[1], state.shape[3]
    o = torch.empty(q.shape[0], H, dv, dtype=torch.float32, device=q.device)
    _mix_ext().gla_recurrence(
        o, q, k, v, z, z_bias, state, slots,
        cu if cu is not None else _empty(positions), positions,
        float(inv_tau), float(q_scale),
    )
    return o


def gated_rmsnorm(o, gate, weight, eps, out_dtype):
    """Per-head RMS norm of o [T, H, dv] (fp32) with a weight shared by heads,
    times silu(gate) -> [T, H*dv] of out_dtype."""
    if not o.is_cuda:
        return ref.gated_rmsnorm(o, gate, weight, eps, out_dtype)
    T, H, dv = o.shape
    out = torch.empty(T, H * dv, dtype=out_dtype, device=o.device)
    _mix_ext().gated_rmsnorm(out, o, gate, weight, float(eps))
    return out


# -- row-cache attention mixers ----------------------------------------------------


def sandwich_rmsnorm(x, y, w_branch, hist, n_hist, dwa, w_next, eps, offset,
                     out_dtype, add_table=None, add_index=None):
    """One residual step of a stack that norms a branch before and after it,
    with an optional weighted average over the outputs of all earlier layers
    (see reference.sandwich_rmsnorm for the exact order of operations). x
    [T, W] fp32 is updated in place; hist [n_max, T, W] fp32; dwa [n_hist]
    fp32. Returns the normed activations in out_dtype, or None."""
    if not x.is_cuda:
        return ref.sandwich_rmsnorm(x, y, w_branch, hist, n_hist, dwa, w_next,
                                    eps, offset, out_dtype, add_table, add_index)
    ext = _mix_ext()
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device) \
        if w_next is not None else _empty(x)
    e = _empty(x)
    ext.sandwich_rmsnorm(
        x, y if y is not None else e, w_branch if y is not None else e,
        hist if hist is not None else e, int(n_hist),
        dwa if dwa is not None else e, w_next if w_next is not None else e,
        float(eps), float(offset), out,
        add_table if add_table is not None else e,
        add_index if add_table is not None else _empty(x, torch.int32),
    )
    return out if w_next is not None else None


def qkv_store(q, k, v, positions, slot_mapping, cache, seg_dim, norm_eps,
              temp_coef, temp_every, q_weight=None, k_weight=None,
              rot_freq=None, rot_mult=1.0, rot_dims=0, norm_whole=False,
              rot_interleaved=False, v_seg=0, v_rot_freq=None, v_cs_out=None):
    """Queries to fp32 (optionally RMS-normed per seg_dim-wide segment, with
    a weight [seg_dim] shared by the segments, or, with norm_whole, over the
    token's whole row with a weight as wide as the row; rotated by position
    on each segment's first rot_dims dimensions (pairs i, i + rot_dims/2, or
    2i, 2i + 1 with rot_interleaved; angles pos * rot_freq[i] in fp32 inside
    the kernel) and multiplied by a position-dependent temperature); keys
    (normed, weighted and rotated alike) and values scattered as one row
    [keys | values] per token into the paged cache. v_rot_freq [v_seg / 2]:
    every v_seg-wide segment of the values is rotated over its whole width
    (same pairing) before it is stored, and v_cs_out [T, v_seg] fp32 receives
    the tokens' (cos, sin) pairs of that rotation (for row_attention's
    out_rot_cs). v None: values = the keys before the norm. k None: no
    store."""
    if not q.is_cuda:
        return ref.qkv_store(q, k, v, positions, slot_mapping, cache, seg_dim,
                             norm_eps, temp_coef, temp_every, q_weight,
                             k_weight, rot_freq, rot_mult, rot_dims,
                             norm_whole, rot_interleaved, v_seg, v_rot_freq,
                             v_cs_out)
    out = torch.empty(q.shape, dtype=torch.float32, device=q.device)
    e = _empty(q)
    ef = _empty(q, torch.float32)
    _mix_ext().qkv_store(
        out, q, k if k is not None else e, v if v is not None else e,
        positions, slot_mapping, cache, int(seg_dim),
        float(norm_eps) if norm_eps is not None else -1.0,
        float(temp_coef), int(temp_every),
        q_weight if q_weight is not None else ef,
        k_weight if k_weight is not None else ef,
        rot_freq if rot_freq is not None else ef, float(rot_mult),
        int(rot_dims) if rot_freq is not None else 0,
        bool(norm_whole), bool(rot_interleaved),
        v_rot_freq if v_rot_freq is not None else ef, int(v_seg),
        v_cs_out if v_cs_out is not None else ef,
    )
    return out


def pool_cache_update(cache, pool, block_tables, token_seq, positions,
                      slot_mapping, pool_tokens):
    """Mean cache row of every block of pool_tokens positions that a token of
    this step completes, into the fp32 pooled rows of its sequence."""
    if not cache.is_cuda:
        return ref.pool_cache_update(cache, pool, block_tables, token_seq,
                                     positions, slot_mapping, pool_tokens)
    _mix_ext().pool_cache_update(
        cache, pool, block_tables,
        token_seq if token_seq is not None else _empty(positions), positions,
        slot_mapping, int(pool_tokens),
    )


def row_attention(q, cache, pool, block_tables, token_seq, positions, heads,
                  kv_heads, maps, dim, vdim, window, pool_tokens, scale,
                  softcap, lam, norm_eps, out_mult, out_dtype, max_seq_len=0,
                  query_bounds=None, head_bias=None, gate=None,
                  shared_kv=False, out_rot_cs=None, out_rot_interleaved=False,
                  value_col=0):
    """Attention of fp32 queries over paged cache rows [keys | values] with
    grouped heads: full causal (window 0) or a sliding window with pooled
    blocks beyond it, optional tanh soft cap, one or two score maps per head
    (two combine as a1 - lam * a2), optional RMS norm of each head's result.
    Key weights: softmax, or, with head_bias [heads] fp32, sigmoid(score +
    head_bias[h]) without normalisation over the keys (one map only). gate
    [T, heads] (fp32 pre-activations): head h's result is multiplied by
    sigmoid(gate[t, h]). max_seq_len: the longest context of the batch as the host
    knows it (0 = the block tables' capacity); it only sizes the split of
    long key ranges over workgroups. query_bounds [B+1] int32 (prompt portions:
    tokens of sequence b are query_bounds[b] .. query_bounds[b+1], at
    consecutive positions) lets the GPU path tile 32 tokens per workgroup on
    the fp32 matrix cores. shared_kv: a cache row holds the keys only (one kv
    head, one map) and the values are its columns value_col .. value_col +
    vdim (vdim == dim: the values are the keys). out_rot_cs [T,
    vdim] fp32 ((cos, sin) per token and pair, as qkv_store's v_cs_out gives
    them): every head's result is turned back by its token's angles over the
    whole value width, in the epilogue of the attention kernel. Returns [T, heads *
    vdim] of out_dtype (the cache's type, or float32)."""
    if not q.is_cuda:
        return ref.row_attention(q, cache, pool, block_tables, token_seq,
                                 positions, heads, kv_heads, maps, dim, vdim,
                                 window, pool_tokens, scale, softcap, lam,
                                 norm_eps, out_mult, out_dtype, head_bias, gate,
                                 shared_kv, out_rot_cs, out_rot_interleaved,
                                 value_col)
    if head_bias is not None and maps != 1:
        raise ValueError("sigmoid key weights take one score map per head")
    out = torch.empty(q.shape[0], heads * vdim, dtype=out_dtype, device=q.device)
    ef = torch.empty(0, dtype=torch.float32, device=q.device)
    _mix_ext().row_attention(
        out, q, cache,
        pool if pool is not None else torch.empty(0, dtype=torch.float32,
                                                  device=q.device),
        block_tables,
        token_seq if token_seq is not None else _empty(positions), positions,
        int(heads), int(kv_heads), int(maps), int(dim), int(vdim), int(window),
        int(pool_tokens), float(scale), float(softcap), float(lam),
        float(norm_eps) if norm_eps is not None else -1.0, float(out_mult),
        int(max_seq_len) or block_tables.shape[1] * cache.shape[1],
        query_bounds if query_bounds is not None and token_seq is not None
        else _empty(positions),
        head_bias if head_bias is not None else ef,
        gate if gate is not None else ef, int(value_col) if shared_kv else -1,
        out_rot_cs if out_rot_cs is not None else ef, bool(out_rot_interleaved),
    )
    return out


def xielu(x, a_pos, a_neg):
    """xIELU activation: a_pos z^2 + z/2 for z > 0, (1/2 + a_neg)(exp(z) - 1 -
    z) + z/2 otherwise (fp32 inside, result in x's dtype)."""
    if not x.is_cuda:
        return ref.xielu(x, a_pos, a_neg)
    out = torch.empty_like(x)
    _mix_ext().xielu(out, x, float(a_pos), float(a_neg))
    return out


# -- post-norm residual stream, minGRU, clamped gated linear unit ----------------


def branch_rmsnorm_add(x, y1, y2, a, b, weight, eps, out_dtype, keep_stream=True):
    """One step of a residual stream that norms a sublayer's OUTPUT, in one
    kernel: y = a * y1 (+ b * y2), x <- x + y / sqrt(mean(y^2) + eps) * weight
    (x None: a new stream that starts as the normed y), everything fp32; x
    [T, W] fp32 is updated in place. y1 / y2 have the activation dtype or fp32.
    Returns (x, x rounded to out_dtype); keep_stream False returns (None, the
    rounded sum) and leaves x as it was."""
    if not y1.is_cuda:
        return ref.branch_rmsnorm_add(x, y1, y2, a, b, weight, eps, out_dtype,
                                      keep_stream)
    ext = _mix_ext()
    T, W = y1.shape
    out = torch.empty(T, W, dtype=out_dtype, device=y1.device)
    x_out = x
    if keep_stream and x is None:
        x_out = torch.empty(T, W, dtype=torch.float32, device=y1.device)
    ef = _empty(y1, torch.float32)
    ext.branch_rmsnorm_add(
        x if x is not None else ef, x_out if keep_stream else ef, y1,
        y2 if y2 is not None else _empty(y1), float(a), float(b), weight,
        float(eps), out,
    )
    return (x_out if keep_stream else None), out


def mingru_scan(zug, z_bias, u_bias, state, slots, cu, positions, out_dtype):
    """minGRU over packed sequences: zug [T, 3 * width] (any row stride) holds
    the pre-activations of update gate, candidate and output gate;
    S_t = S_(t-1) + f (c - S_(t-1)) per channel with f = sigma(z_pre +
    z_bias), p = u_pre + u_bias, c = p + 1/2 where p >= 0 and sigma(p) below. The fp32
    state [slots, width] is read (or started from zero at position 0) and
    written back. cu [B+1] int32 token bounds (None: one token each). Returns
    S_t * silu(g_pre) as [T, width] of out_dtype."""
    if not zug.is_cuda:
        return ref.mingru_scan(zug, z_bias, u_bias, state, slots, cu,
                               positions, out_dtype)
    width = state.shape[1]
    out = torch.empty(zug.shape[0], width, dtype=out_dtype, device=zug.device)
    _mix_ext().mingru_scan(
        out, zug, z_bias, u_bias, state, slots,
        cu if cu is not None else _empty(positions), positions,
    )
    return out


def clamped_glu(gate_up, limit, alpha=1.702):
    """[gate | up] -> a sigma(alpha a) (1 + b), a = gate cut off above at
    `limit`, b = up cut off at -limit and +limit; fp32 inside, result in the
    input dtype."""
    if not gate_up.is_cuda:
        return ref.clamped_glu(gate_up, limit, alpha)
    out = torch.empty(gate_up.shape[0], gate_up.shape[1] // 2,
                      dtype=gate_up.dtype, device=gate_up.device)
    _mix_ext().clamped_glu(out, gate_up, float(limit), float(alpha))
    return out


# -- grouped RMS norm over a parallel residual, hashed pair embedding, relu^2 ----


def group_rmsnorm_add(x, y1, y2, weight, groups, eps, out_dtype):
    """One step of a residual stream whose sublayers all read one norm: x
    [T, W] fp32 <- x + (y1 + y2) in place (y1 None: no update; y2 None: y1
    alone), then the RMS norm in `groups` equal consecutive parts times weight
    -> [T, W] of out_dtype (weight None: no norm, returns None)."""
    if not x.is_cuda:
        return ref.group_rmsnorm_add(x, y1, y2, weight, groups, eps, out_dtype)
    e = _empty(x, out_dtype)
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device) \
        if weight is not None else e
    _mix_ext().group_rmsnorm_add(
        x, y1 if y1 is not None else e, y2 if y2 is not None else e,
        weight if weight is not None else e, int(groups), float(eps), out,
    )
    return out if weight is not None else None


def pair_hash_embedding(ids, prev_ids, table, scale, pair_table, buckets,
                        mul_prev, mul_cur):
    """fp32 [T, W]: table[id] * scale + pair_table[(prev * mul_prev + id *
    mul_cur) mod buckets], or pair_table[buckets] (its last row) where a token
    has no predecessor (prev < 0). ids, prev_ids [T] int64."""
    if not table.is_cuda:
        return ref.pair_hash_embedding(ids, prev_ids, table, scale, pair_table,
                                       buckets, mul_prev, mul_cur)
    out = torch.empty(ids.shape[0], table.shape[1], dtype=torch.float32,
                      device=table.device)
    _mix_ext().pair_hash_embedding(out, ids, prev_ids, table, pair_table,
                                   float(scale), int(buckets), int(mul_prev),
                                   int(mul_cur))
    return out


def relu_squared(x):
    """max(x, 0)^2; x [rows, I] may be a column range of a wider matrix."""
    if not x.is_cuda:
        return ref.relu_squared(x)
    out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    _mix_ext().relu_squared(out, x)
    return out


def rotate_heads(x, positions, freq, interleaved, sign, out_dtype):
    """x [T, H, D] fp32: every head turned over its whole width by sign * pos
    * freq[m] (pair m = dimensions m, m + D/2, or 2m, 2m + 1 when interleaved;
    angles in fp32). Returns [T, H * D] of out_dtype."""
    if not x.is_cuda:
        return ref.rotate_heads(x, positions, freq, interleaved, sign, out_dtype)
    T, H, D = x.shape
    out = torch.empty(T, H * D, dtype=out_dtype, device=x.device)
    _mix_ext().rotate_heads(out, x.contiguous(), freq, positions,
                            bool(interleaved), float(sign))
    return out

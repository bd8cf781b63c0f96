"""Python launchers of the ragged-batch serving kernels (csrc/seqmix.hip, csrc/bgemm.hip, csrc/latent_attn.hip, csrc/seqrec.hip, csrc/seqsand.hip): hashed-bigram embedding,
post-sum LayerNorm on an fp32 residual stream, latent key/value rows, rotary embedding in both pair layouts, two-part-key / grouped-query / windowed attention,
gated linear attention and retention with carried state, the sigmoid and softmax routers and the grouped expert products (with gated epilogues), the residual
sum with RMS norms in groups, short convolutions with carried inputs, query / key / value rows into a slot cache, the gated delta rule, gated activations,
the residual sum between two norms (sandwich norms), pooled key / value rows, xIELU and sigmoid output gates on rows.

Activations are bf16 (serving mode: bf16 operands, fp32 accumulation) or fp32 (true 32-bit mode: every product is an fp32 FMA chain; the bf16
weights are exactly representable and widened on load).  Whatever the mode, the residual stream, norm statistics, rotary angles, decays,
recurrent state and the router are fp32.  There is no CPU path.
"""

import torch

from . import _lib as L
from . import kernels as K

BF16, F32, I32 = torch.bfloat16, torch.float32, torch.int32


def _dt(t):
    return L.dt_code(t.dtype)


def _rows(t, name):
    if t.dim() != 2 or t.stride(1) != 1:
        raise ValueError(f"{name}: a 2-D tensor with unit inner stride is required, got shape {tuple(t.shape)} strides {t.stride()}")


def _i32(t, name, n=None):
    if t.dtype != I32 or not t.is_contiguous() or (n is not None and t.numel() < n):
        raise ValueError(f"{name}: contiguous int32 tensor{'' if n is None else f' of at least {n} entries'} required")


def embed_hash(tok, prev, table, scale, bigram=None, buckets=0, mul_prev=0, mul_cur=0):
    """fp32 [tokens, width] = table[tok] * scale (+ bigram row hashed from (prev, tok); prev < 0 selects row ``buckets``)."""
    L.require_gpu(tok, prev, table, bigram)
    T = tok.numel()
    _i32(tok, "embed_hash(tok)")
    if bigram is not None:
        _i32(prev, "embed_hash(prev)", T)
        if bigram.dtype != BF16 or not bigram.is_contiguous() or tuple(bigram.shape) != (buckets + 1, table.shape[1]):
            raise ValueError("embed_hash: the bigram table is bf16 [buckets + 1, width]")
    if table.dtype != BF16 or not table.is_contiguous():
        raise ValueError("embed_hash: the table is contiguous bf16")
    out = torch.empty((T, table.shape[1]), dtype=F32, device=table.device)
    L.call("mi355_embed_hash_fwd", T, table.shape[1], table.shape[0], L.ptr(tok), L.ptr(prev), L.ptr(table), float(scale), L.ptr(bigram), int(buckets),
           int(mul_prev), int(mul_cur), L.ptr(out))
    return out


def add_layernorm(x, w, b, eps, alpha=1.0, y=None, parts=1, cast_dtype=None):
    """LayerNorm(alpha * x + sum of y's ``parts`` rows per token) on fp32 rows -> (fp32 rows, the same rows in ``cast_dtype`` or None)."""
    L.require_gpu(x, w, b, y)
    _rows(x, "add_layernorm(x)")
    T, width = x.shape
    if x.dtype != F32 or not x.is_contiguous() or w.dtype != F32 or b.dtype != F32 or w.numel() != width or b.numel() != width:
        raise ValueError("add_layernorm: x contiguous fp32 [tokens, width], weight and bias fp32 [width]")
    if y is not None:
        _rows(y, "add_layernorm(y)")
        if y.shape[0] != T * parts or y.shape[1] != width:
            raise ValueError(f"add_layernorm: the summand must be [{T * parts}, {width}], got {tuple(y.shape)}")
    out = torch.empty_like(x)
    cast = None if cast_dtype is None or cast_dtype == F32 else torch.empty((T, width), dtype=cast_dtype, device=x.device)
    L.call("mi355_add_layernorm_fwd", T, width, L.ptr(x), float(alpha), L.ptr(y), 0 if y is None else _dt(y), 0 if y is None else y.stride(0), int(parts),
           L.ptr(w), L.ptr(b), float(eps), L.ptr(out), L.ptr(cast), 0 if cast is None else _dt(cast))
    return out, (out if cast_dtype == F32 else cast)


def rmsnorm_rows(x, w, eps, out_dtype=None):
    L.require_gpu(x, w)
    _rows(x, "rmsnorm_rows(x)")
    if w.dtype != F32 or w.numel() != x.shape[1]:
        raise ValueError("rmsnorm_rows: weight fp32 [n]")
    out = torch.empty(x.shape, dtype=out_dtype or x.dtype, device=x.device)
    L.call("mi355_rmsnorm_rows", x.shape[0], x.shape[1], L.ptr(x), _dt(x), x.stride(0), L.ptr(w), float(eps), L.ptr(out), _dt(out), out.stride(0))
    return out


def rope_frequencies(dims, base, device):
    """fp32 [dims / 2]: base^(-2i / dims), evaluated in double."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    return torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / dims).to(F32).to(device)


def latent_kv_append(src, rank, rot, w, eps, pos, dst_row, freq, dims, cache2d, layout=0):
    """src [tokens, rank + rot] -> rows ``dst_row`` of ``cache2d`` [rows, rank + rot]: RMSNorm on the latent, rotary on the shared key part (``layout`` 0:
    neighbouring entries form a pair; 1: entry i pairs with entry i + dims / 2)."""
    L.require_gpu(src, w, pos, dst_row, freq, cache2d)
    _rows(src, "latent_kv_append(src)")
    _rows(cache2d, "latent_kv_append(cache)")
    T = src.shape[0]
    _i32(pos, "latent_kv_append(pos)", T)
    _i32(dst_row, "latent_kv_append(dst_row)", T)
    if src.shape[1] != rank + rot or cache2d.shape[1] != rank + rot or w.dtype != F32 or w.numel() != rank or (dims and (freq.dtype != F32 or freq.numel() < dims // 2)):
        raise ValueError("latent_kv_append: operand sizes do not match rank / rot")
    L.call("mi355_latent_kv_append", T, rank, rot, L.ptr(src), _dt(src), src.stride(0), L.ptr(w), float(eps), L.ptr(pos), L.ptr(dst_row), L.ptr(freq), int(dims),
           int(layout), L.ptr(cache2d), _dt(cache2d), cache2d.stride(0))


def rope_heads(src, H, n, src_hs, src_off, dst, dst_hs, dst_off, rot_start, dims, freq, pos, layout=0):
    """dst (fp32) <- n entries per head of src, the pairs of [rot_start, rot_start + dims) rotated by the token's position.  ``layout`` 0: neighbouring
    entries form a pair; 1: entry i pairs with entry i + dims / 2."""
    L.require_gpu(src, dst, freq, pos)
    _rows(src, "rope_heads(src)")
    _rows(dst, "rope_heads(dst)")
    if dst.dtype != F32 or dst.shape[0] != src.shape[0]:
        raise ValueError("rope_heads: dst is fp32 with src's rows")
    _i32(pos, "rope_heads(pos)", src.shape[0])
    if src.shape[1] < (H - 1) * src_hs + src_off + n or dst.shape[1] < (H - 1) * dst_hs + dst_off + n:
        raise ValueError("rope_heads: rows too short for the head layout")
    L.call("mi355_rope_heads", src.shape[0], H, n, L.ptr(src), _dt(src), src.stride(0), src_hs, src_off, L.ptr(dst), dst.stride(0), dst_hs, dst_off, rot_start, dims,
           int(layout), L.ptr(freq), L.ptr(pos))
    return dst


def gated_headnorm(o, w, gate, H, D, eps, out_dtype):
    L.require_gpu(o, w, gate)
    _rows(gate, "gated_headnorm(gate)")
    if o.dtype != F32 or not o.is_contiguous() or o.shape[1] != H * D or gate.shape != o.shape or w.dtype != F32 or w.numel() != D:
        raise ValueError("gated_headnorm: o contiguous fp32 [tokens, H*D], gate a view of that shape, weight fp32 [D]")
    out = torch.empty(o.shape, dtype=out_dtype, device=o.device)
    L.call("mi355_gated_headnorm", o.shape[0], H, D, L.ptr(o), L.ptr(w), L.ptr(gate), _dt(gate), gate.stride(0), float(eps), L.ptr(out), _dt(out), out.stride(0))
    return out


def gla(q, k, v, z, zbias, inv_tau, qscale, seq_off, slot, state, H, dk, dv, head_decay=None, kscale=1.0):
    """Gated linear attention over a ragged batch; ``state`` fp32 [slots, H, dk, dv] is read and written at ``slot``.  Returns fp32 [tokens, H * dv].
    ``head_decay`` (fp32 [H]): a fixed decay per head instead of the per-channel one from ``z`` (``z`` / ``zbias`` may then be None); keys are multiplied
    by ``kscale``."""
    L.require_gpu(q, k, v, z, zbias, seq_off, slot, state, head_decay)
    if head_decay is not None:
        if head_decay.dtype != F32 or not head_decay.is_contiguous() or head_decay.numel() != H:
            raise ValueError("gla: head_decay fp32 [H]")
        return _gla_fixed(q, k, v, head_decay, qscale, kscale, seq_off, slot, state, H, dk, dv)
    for t, n, w in ((q, "q", H * dk), (k, "k", H * dk), (z, "z", H * dk), (v, "v", H * dv)):
        _rows(t, f"gla({n})")
        if t.shape[1] != w or (n != "z" and t.dtype != q.dtype) or t.shape[0] != q.shape[0]:
            raise ValueError(f"gla({n}): [tokens, {w}] of q's dtype required")
    n_seq = slot.numel()
    _i32(seq_off, "gla(seq_off)", n_seq + 1)
    _i32(slot, "gla(slot)")
    if state.dtype != F32 or not state.is_contiguous() or tuple(state.shape[1:]) != (H, dk, dv) or zbias.dtype != F32 or zbias.numel() != H * dk:
        raise ValueError("gla: state fp32 [slots, H, dk, dv], bias fp32 [H * dk]")
    o = torch.empty((q.shape[0], H * dv), dtype=F32, device=q.device)
    L.call("mi355_gla_fwd", n_seq, L.ptr(seq_off), L.ptr(slot), H, dk, dv, L.ptr(q), L.ptr(k), L.ptr(v), L.ptr(z), _dt(q), _dt(z), _dt(v), q.stride(0), k.stride(0), v.stride(0),
           z.stride(0), L.ptr(zbias), float(inv_tau), float(qscale), None, float(kscale), L.ptr(state), L.ptr(o))
    return o


def _gla_fixed(q, k, v, head_decay, qscale, kscale, seq_off, slot, state, H, dk, dv):
    for t, n, w in ((q, "q", H * dk), (k, "k", H * dk), (v, "v", H * dv)):
        _rows(t, f"gla({n})")
        if t.shape[1] != w or (n != "v" and t.dtype != q.dtype) or t.shape[0] != q.shape[0]:
            raise ValueError(f"gla({n}): [tokens, {w}] required (k of q's dtype)")
    n_seq = slot.numel()
    _i32(seq_off, "gla(seq_off)", n_seq + 1)
    _i32(slot, "gla(slot)")
    if state.dtype != F32 or not state.is_contiguous() or tuple(state.shape[1:]) != (H, dk, dv):
        raise ValueError("gla: state fp32 [slots, H, dk, dv]")
    o = torch.empty((q.shape[0], H * dv), dtype=F32, device=q.device)
    L.call("mi355_gla_fwd", n_seq, L.ptr(seq_off), L.ptr(slot), H, dk, dv, L.ptr(q), L.ptr(k), L.ptr(v), None, _dt(q), 0, _dt(v), q.stride(0), k.stride(0), v.stride(0),
           0, None, 1.0, float(qscale), L.ptr(head_decay), float(kscale), L.ptr(state), L.ptr(o))
    return o


def router_logits(x32, w):
    """fp32 [tokens, experts] = x32 (fp32 rows) times w[experts, width]^T (bf16), fp32 FMA."""
    L.require_gpu(x32, w)
    _rows(x32, "router_logits(x)")
    if x32.dtype != F32 or w.dtype != BF16 or w.dim() != 2 or w.stride(1) != 1 or w.shape[1] != x32.shape[1]:
        raise ValueError("router_logits: x fp32 [tokens, width], w bf16 [experts, width]")
    out = torch.empty((x32.shape[0], w.shape[0]), dtype=F32, device=x32.device)
    L.call("mi355_router_logits", x32.shape[0], w.shape[0], w.shape[1], L.ptr(x32), x32.stride(0), L.ptr(w), w.stride(0), L.ptr(out))
    return out


def moe_route(logits, correction, top, groups, keep, scale, softmax=False):
    """(ids int32 [tokens, top], weights fp32 [tokens, top]).  ``softmax`` True: scores are the softmax over all experts, the winners' scores times ``scale``
    are the weights (not renormalised); ``softmax`` "chosen": ``correction`` is a bias on the logits, the ``top`` largest win and their weights are the
    softmax over the winners' logits alone (times ``scale``); otherwise the grouped sigmoid router."""
    L.require_gpu(logits, correction)
    if logits.dtype != F32 or not logits.is_contiguous() or (correction is not None and (correction.dtype != F32 or correction.numel() != logits.shape[1])):
        raise ValueError("moe_route: logits contiguous fp32 [tokens, experts], correction fp32 [experts]")
    T, E = logits.shape
    ids = torch.empty((T, top), dtype=I32, device=logits.device)
    wts = torch.empty((T, top), dtype=F32, device=logits.device)
    L.call("mi355_moe_route", T, E, top, groups, keep, L.ptr(logits), L.ptr(correction), float(scale), 2 if softmax == "chosen" else 1 if softmax else 0, L.ptr(ids), L.ptr(wts))
    return ids, wts


def moe_dispatch(ids, E):
    L.require_gpu(ids)
    _i32(ids, "moe_dispatch(ids)")
    offs = torch.empty((E + 1,), dtype=I32, device=ids.device)
    perm = torch.empty((ids.numel(),), dtype=I32, device=ids.device)
    L.call("mi355_moe_dispatch", ids.numel(), E, L.ptr(ids), L.ptr(offs), L.ptr(perm))
    return offs, perm


def bgemm(a, b, c, M, N, Kd, batch=1, lda=None, a_bs=0, sbn=None, sbk=1, b_bs=0, ldc=None, c_bs=0, grp_offs=None, a_rows=None, a_div=1, c_rows=None,
          row_scale=None, epi=0, mfma=None, bias=None, limit=0.0, n_out=0):
    """The general strided product (see include/mi355_vlm.h).  Strides default to a's / c's row pitch and b stored [N, K]; the caller vouches that the
    strides stay inside the tensors.  ``mfma`` defaults to bf16 a and b."""
    L.require_gpu(a, b, c, grp_offs, a_rows, c_rows, row_scale, bias)
    if bias is not None and (bias.dtype != F32 or not bias.is_contiguous() or bias.numel() != N):
        raise ValueError("bgemm: bias contiguous fp32 [N]")
    if mfma is None:
        mfma = a.dtype == BF16 and b.dtype == BF16
    L.call("mi355_bgemm", batch, M, N, Kd, L.ptr(a), _dt(a), a.stride(0) if lda is None else lda, a_bs, L.ptr(b), _dt(b), b.stride(0) if sbn is None else sbn, sbk, b_bs,
           L.ptr(c), _dt(c), c.stride(0) if ldc is None else ldc, c_bs, L.ptr(grp_offs), L.ptr(a_rows), a_div, L.ptr(c_rows), L.ptr(row_scale), epi, 1 if mfma else 0, L.ptr(bias), float(limit), int(n_out))
    return c


def linear(x, w, out_dtype=None, bias=None):
    """x [M, K] (bf16 or fp32) times w[N, K]^T (bf16) (+ bias fp32 [N]).  bf16 rows go through the MFMA GEMMs (weight stream for <= 8 rows), fp32 rows through
    the fp32 FMA product."""
    _rows(x, "linear(x)")
    M, Kd = x.shape
    N = w.shape[0]
    if w.dtype != BF16 or w.shape[1] != Kd or w.stride(1) != 1:
        raise ValueError("linear: weight bf16 [N, K] with unit inner stride")
    out_dtype = out_dtype or x.dtype
    if x.dtype == BF16:
        aligned = Kd % 8 == 0 and x.stride(0) % 8 == 0 and w.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0
        if aligned and M <= 8 and out_dtype == BF16 and bias is None:
            from . import ops_decode

            return ops_decode.gemv(x, w)
        if aligned and M <= 8 and out_dtype == F32 and (bias is None or (bias.dtype == F32 and bias.is_contiguous() and bias.numel() == N)):
            L.require_gpu(x, w, bias)
            out = torch.empty((M, N), dtype=F32, device=x.device)
            L.call("mi355_gemv_bf16_f32out", M, N, Kd, L.ptr(x), x.stride(0), L.ptr(w), w.stride(0), L.ptr(out), out.stride(0), L.ptr(bias))
            return out
        if aligned and M > 8:
            return K.gemm(L.GEMM_NT, x, w, out_dtype=out_dtype, bias=bias)
    out = torch.empty((M, N), dtype=out_dtype, device=x.device)
    return bgemm(x, w, out, M, N, Kd, bias=bias)


def attn_key_splits(n_seq, head_tiles, max_new, hm, max_keys, per_split=256):
    """Workgroups per tile of the MFMA attention: a step with few query tiles and long caches (one-token steps) deals each tile's keys to several, about
    ``per_split`` keys each, as many as fill the chip's 256 CUs once."""
    tiles = n_seq * head_tiles * -(-max_new * hm // 128)
    if max_keys <= 2 * per_split or tiles >= 128:
        return 1
    return max(1, min(-(-max_keys // per_split), 32, 256 // tiles))


def latent_attn(q, k1, k2, v, out, H, hm, D1, D2, DV, q_hs, k1_hs, v_hs, o_hs, desc, max_new, scale, max_keys=0, kv_rep=1, window=0, keep_first=0, softcap=0.0,
                sink=None, pool=0, pooled=None, pool_row0=None, chunk=0):
    """Two-part-key causal attention over a ragged batch.  ``desc`` = (q_row0, n_new, past, k1_row0, k2_row0, v_row0) int32 [n_seq] each.  ``max_keys``
    (the longest sequence's keys, if the caller knows it) lets one-token steps over long caches spread a tile's keys over several workgroups.
    ``kv_rep``: query heads per key / value head (strides per key / value head).  ``window`` > 0: a query sees a key only ``window`` positions back, or
    among the first ``keep_first`` of the sequence.  ``softcap`` > 0: scores pass cap * tanh(score / cap).  ``sink`` (fp32 [H]): exp(sink[h]) joins head h's
    denominator.  ``pool`` > 0: ``pooled`` = (pooled keys, pooled values), views laid out like ``k1`` / ``v`` with one mean row per ``pool`` tokens, first row
    of every sequence in ``pool_row0`` (int32 [n_seq]); a query sees the blocks that lie wholly before its window.  ``chunk`` > 0: positions are cut into chunks
    of that many from the sequence's first token on, and a query sees only the keys of its own chunk."""
    L.require_gpu(q, k1, k2, v, out, sink, pool_row0, *desc)
    pk = pv = None
    if pool:
        pk, pv = pooled
        L.require_gpu(q, pk, pv)
        _rows(pk, "latent_attn(pooled keys)")
        _rows(pv, "latent_attn(pooled values)")
        _i32(pool_row0, "latent_attn(pool_row0)", desc[0].numel())
        if pk.dtype != v.dtype or pv.dtype != v.dtype or pk.stride(0) != pv.stride(0):
            raise ValueError("latent_attn: pooled rows share the dtype of keys / values and one row pitch")
    if sink is not None and (sink.dtype != F32 or not sink.is_contiguous() or sink.numel() != H):
        raise ValueError("latent_attn: sink fp32 [H]")
    for t, n in ((q, "q"), (k1, "k1"), (v, "v"), (out, "out")):
        _rows(t, f"latent_attn({n})")
    if q.dtype != F32 or k1.dtype != v.dtype or out.dtype != v.dtype or (k2 is not None and k2.dtype != v.dtype):
        raise ValueError("latent_attn: q fp32; keys, values and output share one dtype")
    n_seq = desc[0].numel()
    for t in desc:
        _i32(t, "latent_attn(desc)", n_seq)
    mfma = v.dtype == BF16
    splits, ws = 1, None
    # A plain window leaves a tile window + its own tokens to see: that range is dealt out, in finer shares (a one-token step over it is a chain of
    # dependent 64-key steps in very few workgroups).  A window that also keeps the first tokens is not dealt out: the kernel skips what lies between.
    plain_window = window and window < max_keys and not keep_first
    reach = min(window or chunk, chunk or window)  # the most keys a row sees besides those of its own tile
    if chunk and chunk < max_keys and not keep_first:
        plain_window = True
    if mfma and D1 + D2 <= 320 and DV <= 256 and max_keys and (not window or window >= max_keys or plain_window):
        head_tiles = -(-H // hm)
        tile_tokens = min(max_new, -(-128 // hm))
        if plain_window:  # what a tile walks: its window, and one pooled row per block before it
            rows = min(max_keys, reach + tile_tokens - 1) + (max(0, max_keys - window) // pool if pool else 0)
            splits = attn_key_splits(n_seq, head_tiles, max_new, hm, rows, 128)
        else:
            splits = attn_key_splits(n_seq, head_tiles, max_new, hm, max_keys)
        if splits > 1:
            dvp = 32 if DV <= 32 else 64 if DV <= 64 else 128 if DV <= 128 else 256
            ws = torch.empty(n_seq * head_tiles * -(-max_new * hm // 128) * splits * 128 * (2 + dvp), dtype=F32, device=v.device)
    L.call("mi355_latent_attn", n_seq, max_new, H, hm, D1, D2, DV, L.ptr(q), q.stride(0), q_hs, L.ptr(k1), k1.stride(0), k1_hs, L.ptr(k2), 0 if k2 is None else k2.stride(0),
           L.ptr(v), v.stride(0), v_hs, L.ptr(out), out.stride(0), o_hs, _dt(v), *[L.ptr(t) for t in desc], float(scale), 1 if mfma else 0, splits, L.ptr(ws),
           0 if ws is None else ws.numel(), int(kv_rep), int(window), int(keep_first), float(softcap or 0.0), L.ptr(sink), int(pool), L.ptr(pk), L.ptr(pv),
           0 if pk is None else pk.stride(0), L.ptr(pool_row0), int(chunk))
    return out


def group_rmsnorm_sum(x, groups, eps, y1=None, y2=None, parts=1, x_out=None, norm_a=None, norm_b=None):
    """v = x + y1 + (sum of y2's ``parts`` rows per token) on fp32 rows; ``x_out`` (True: a new tensor, or a tensor, or None) receives v.  ``norm_a`` /
    ``norm_b`` = (weight fp32 [width], dtype or None, want_fp32_copy): RMS norm of v in ``groups`` equal consecutive groups times the weight.
    Returns (x_out or None, (a, a32), (b, b32))."""
    L.require_gpu(x, y1, y2)
    _rows(x, "group_rmsnorm_sum(x)")
    T, width = x.shape
    if x.dtype != F32 or not x.is_contiguous():
        raise ValueError("group_rmsnorm_sum: x contiguous fp32 [tokens, width]")
    for y, n, rows in ((y1, "y1", T), (y2, "y2", T * parts)):
        if y is not None:
            _rows(y, f"group_rmsnorm_sum({n})")
            if tuple(y.shape) != (rows, width):
                raise ValueError(f"group_rmsnorm_sum({n}): [{rows}, {width}] required, got {tuple(y.shape)}")
    if x_out is True:
        x_out = torch.empty_like(x)
    outs, args = [], []
    for nm in (norm_a, norm_b):
        if nm is None:
            outs.append((None, None))
            args += [None, None, 0, None]
            continue
        w, dtype, want32 = nm
        if w.dtype != F32 or w.numel() != width or not w.is_contiguous():
            raise ValueError("group_rmsnorm_sum: weight fp32 [width]")
        o = torch.empty((T, width), dtype=dtype, device=x.device) if dtype is not None else None
        o32 = o if dtype == F32 and want32 else (torch.empty((T, width), dtype=F32, device=x.device) if want32 else None)
        outs.append((o, o32))
        args += [L.ptr(w), L.ptr(o), 0 if o is None else _dt(o), None if o32 is o else L.ptr(o32)]
    L.call("mi355_group_rmsnorm_sum", T, width, L.ptr(x), L.ptr(y1), 0 if y1 is None else _dt(y1), 0 if y1 is None else y1.stride(0), L.ptr(y2),
           0 if y2 is None else _dt(y2), 0 if y2 is None else y2.stride(0), int(parts), L.ptr(x_out), int(groups), float(eps), *args)
    return x_out, outs[0], outs[1]


def ragged_conv(x, w, state, row_seq, seq_off, slot, act=False, residual=False, out_dtype=None, bias=None):
    """Causal convolution over time on every channel of the packed rows ``x`` [tokens, C], w fp32 [C, taps]; ``state`` fp32 [slots, taps - 1, C] carries a
    sequence's last inputs from step to step (read, then updated).  y = (x if residual) + (silu if act)(conv + bias)."""
    L.require_gpu(x, w, state, row_seq, seq_off, slot, bias)
    if bias is not None and (bias.dtype != F32 or not bias.is_contiguous() or bias.numel() != x.shape[1]):
        raise ValueError("ragged_conv: bias contiguous fp32 [C]")
    _rows(x, "ragged_conv(x)")
    T, C = x.shape
    taps = w.shape[1]
    n_seq = slot.numel()
    if w.dtype != F32 or not w.is_contiguous() or w.shape[0] != C:
        raise ValueError("ragged_conv: weight contiguous fp32 [C, taps]")
    if taps > 1 and (state is None or state.dtype != F32 or not state.is_contiguous() or tuple(state.shape[1:]) != (taps - 1, C)):
        raise ValueError("ragged_conv: state contiguous fp32 [slots, taps - 1, C]")
    _i32(row_seq, "ragged_conv(row_seq)", T)
    _i32(seq_off, "ragged_conv(seq_off)", n_seq + 1)
    _i32(slot, "ragged_conv(slot)")
    y = torch.empty((T, C), dtype=out_dtype or x.dtype, device=x.device)
    L.call("mi355_ragged_conv", T, n_seq, C, taps, L.ptr(x), _dt(x), x.stride(0), L.ptr(w), L.ptr(row_seq), L.ptr(seq_off), L.ptr(slot), L.ptr(state), 1 if act else 0,
           1 if residual else 0, L.ptr(y), _dt(y), y.stride(0), L.ptr(bias))
    return y


def qkv_rows_append(src, H, G, d, dv, bias, qw, kw, eps, qscale, dims, layout, freq, pos, dst_row, cache2d, q_temp=None, vmix=None, lam=0.0):
    """Rows [H x d | G x d | G x dv] -> fp32 queries [tokens, H * d] (bias, head norm, rotation, per-head scale) and key / value rows of ``cache2d``.
    ``q_temp`` = (coef, every): the query at position p is also multiplied by 1 + coef * ln(floor((p + 1) / every) + 1).  ``vmix`` (fp32 [tokens, G * dv],
    any row pitch): the cached value is (1 - lam) v + lam * vmix."""
    L.require_gpu(src, bias, qw, kw, qscale, freq, pos, dst_row, cache2d, vmix)
    if vmix is not None:
        _rows(vmix, "qkv_rows_append(vmix)")
        if vmix.dtype != F32 or tuple(vmix.shape) != (src.shape[0], G * dv):
            raise ValueError(f"qkv_rows_append: the rows to mix in are fp32 [{src.shape[0]}, {G * dv}]")
    coef, every = (float(q_temp[0]), int(q_temp[1])) if q_temp else (0.0, 0)
    if q_temp and every < 1:
        raise ValueError("qkv_rows_append: the query temperature's step is a positive number of positions")
    _rows(src, "qkv_rows_append(src)")
    _rows(cache2d, "qkv_rows_append(cache)")
    T = src.shape[0]
    if src.shape[1] != (H + G) * d + G * dv or cache2d.shape[1] != G * (d + dv):
        raise ValueError("qkv_rows_append: row widths do not match the head layout")
    for t, n in ((bias, (H + G) * d + G * dv), (qw, d), (kw, d), (qscale, H), (freq, dims // 2)):
        if t is not None and (t.dtype != F32 or not t.is_contiguous() or t.numel() < n):
            raise ValueError("qkv_rows_append: vectors are contiguous fp32 of the layout's sizes")
    _i32(pos, "qkv_rows_append(pos)", T)
    _i32(dst_row, "qkv_rows_append(dst_row)", T)
    q = torch.empty((T, H * d), dtype=F32, device=src.device)
    L.call("mi355_qkv_rows_append", T, H, G, d, dv, L.ptr(src), _dt(src), src.stride(0), L.ptr(bias), L.ptr(qw), L.ptr(kw), float(eps), L.ptr(qscale), int(dims), int(layout),
           L.ptr(freq), L.ptr(pos), L.ptr(dst_row), L.ptr(q), q.stride(0), L.ptr(cache2d), _dt(cache2d), cache2d.stride(0), coef, every, L.ptr(vmix),
           0 if vmix is None else vmix.stride(0), float(lam))
    return q


def delta_rule(q, k, v, b, a, A_log, dt_bias, qscale, seq_off, slot, state, H, G, dk, dv):
    """Gated delta rule over a ragged batch (raw q / k rows: made unit vectors inside); ``state`` fp32 [slots, H, dk, dv].  Returns fp32 [tokens, H * dv]."""
    L.require_gpu(q, k, v, b, a, A_log, dt_bias, seq_off, slot, state)
    T = q.shape[0]
    for t, n, w in ((q, "q", G * dk), (k, "k", G * dk), (v, "v", H * dv), (b, "b", H), (a, "a", H)):
        _rows(t, f"delta_rule({n})")
        if t.shape != (T, w):
            raise ValueError(f"delta_rule({n}): [tokens, {w}] required")
    if q.dtype != k.dtype or b.dtype != a.dtype:
        raise ValueError("delta_rule: q / k share a dtype, so do b / a")
    n_seq = slot.numel()
    _i32(seq_off, "delta_rule(seq_off)", n_seq + 1)
    _i32(slot, "delta_rule(slot)")
    if state.dtype != F32 or not state.is_contiguous() or tuple(state.shape[1:]) != (H, dk, dv):
        raise ValueError("delta_rule: state fp32 [slots, H, dk, dv]")
    for t in (A_log, dt_bias):
        if t.dtype != F32 or t.numel() != H or not t.is_contiguous():
            raise ValueError("delta_rule: A_log and dt_bias fp32 [H]")
    o = torch.empty((T, H * dv), dtype=F32, device=q.device)
    ws = torch.empty((T * H * 4,), dtype=F32, device=q.device)  # per token and head: decay, beta, the two unit-vector factors
    L.call("mi355_delta_rule_ragged", T, n_seq, L.ptr(seq_off), L.ptr(slot), H, G, dk, dv, L.ptr(q), L.ptr(k), _dt(q), q.stride(0), k.stride(0), L.ptr(v), _dt(v), v.stride(0),
           L.ptr(b), L.ptr(a), _dt(b), b.stride(0), a.stride(0), L.ptr(A_log), L.ptr(dt_bias), float(qscale), L.ptr(state), L.ptr(o), L.ptr(ws))
    return o


GLU_GELU_TANH, GLU_CLAMPED_SWISH, GLU_SILU = 0, 1, 2
EPI_RELU2, EPI_CLAMPED_SWISH_GLU, EPI_GELU_TANH_GLU, EPI_SILU_GLU = 1, 2, 3, 4  # epilogues of bgemm


def pack_gate_up(gate, up):
    """[F, K] gate and up weights -> [64 * ceil(F / 32), K]: blocks of 32 gate rows followed by their 32 up rows (zero rows pad the last block), the
    layout the gated epilogues of ``bgemm`` read -- a lane of the product then holds a gate and its up."""
    F, Kd = gate.shape
    nb = -(-F // 32)
    out = gate.new_zeros((nb, 2, 32, Kd))
    pad = nb * 32 - F
    g = torch.cat([gate, gate.new_zeros((pad, Kd))]) if pad else gate
    u = torch.cat([up, up.new_zeros((pad, Kd))]) if pad else up
    out[:, 0] = g.reshape(nb, 32, Kd)
    out[:, 1] = u.reshape(nb, 32, Kd)
    return out.reshape(nb * 64, Kd)


def glu_rows(x, kind, limit=0.0, out_dtype=None):
    """Rows [gate | up] -> act(gate) * up: ``GLU_GELU_TANH``, ``GLU_SILU``, or ``GLU_CLAMPED_SWISH`` (g = min(gate, limit), u = clamp(up, +-limit),
    g sigmoid(1.702 g) (u + 1))."""
    L.require_gpu(x)
    _rows(x, "glu_rows(x)")
    F = x.shape[1] // 2
    out = torch.empty((x.shape[0], F), dtype=out_dtype or x.dtype, device=x.device)
    L.call("mi355_glu_rows", x.shape[0], F, L.ptr(x), _dt(x), x.stride(0), int(kind), float(limit), L.ptr(out), _dt(out), out.stride(0))
    return out


def sandwich_rmsnorm(x, eps, y=None, w_post=None, w_next=None, out_dtype=None, x_out=None):
    """The residual sum between two norms: v = x + RMSNorm(y) * w_post (``y`` None: v = x); ``x_out`` (True: a new tensor; or x itself; or None) receives v;
    with ``w_next`` the normed row RMSNorm(v) * w_next is returned in ``out_dtype``.  x fp32, weights fp32 [width].  Returns (x_out or None, normed or None)."""
    L.require_gpu(x, y, w_post, w_next)
    _rows(x, "sandwich_rmsnorm(x)")
    T, width = x.shape
    if x.dtype != F32 or not x.is_contiguous():
        raise ValueError("sandwich_rmsnorm: x contiguous fp32 [tokens, width]")
    if y is not None:
        _rows(y, "sandwich_rmsnorm(y)")
        if tuple(y.shape) != (T, width) or w_post is None:
            raise ValueError(f"sandwich_rmsnorm: the sublayer output is [{T}, {width}] and comes with its norm weight")
    for w in (w_post, w_next):
        if w is not None and (w.dtype != F32 or w.numel() != width or not w.is_contiguous()):
            raise ValueError("sandwich_rmsnorm: weight fp32 [width]")
    if x_out is True:
        x_out = torch.empty_like(x)
    out = torch.empty((T, width), dtype=out_dtype or F32, device=x.device) if w_next is not None else None
    L.call("mi355_sandwich_rmsnorm", T, width, L.ptr(x), L.ptr(y), 0 if y is None else _dt(y), 0 if y is None else y.stride(0), L.ptr(w_post), L.ptr(x_out), L.ptr(w_next),
           float(eps), L.ptr(out), 0 if out is None else _dt(out))
    return x_out, out


def pool_rows_update(cache2d, pooled2d, pool, cache_row0, pool_row0, past, n_new, max_blocks):
    """Every block of ``pool`` cache rows that this step completed gets its mean row in ``pooled2d`` (block b of sequence s = row pool_row0[s] + b).
    ``max_blocks``: the most blocks one sequence completes in this step (the host knows the lengths); 0 launches nothing."""
    if max_blocks <= 0:
        return
    L.require_gpu(cache2d, pooled2d, cache_row0, pool_row0, past, n_new)
    _rows(cache2d, "pool_rows_update(cache)")
    _rows(pooled2d, "pool_rows_update(pooled)")
    n_seq = past.numel()
    for t in (cache_row0, pool_row0, past, n_new):
        _i32(t, "pool_rows_update(desc)", n_seq)
    if cache2d.shape[1] != pooled2d.shape[1]:
        raise ValueError("pool_rows_update: pooled rows are as wide as the cache rows")
    L.call("mi355_pool_rows_update", n_seq, int(max_blocks), cache2d.shape[1], int(pool), L.ptr(cache2d), _dt(cache2d), cache2d.stride(0), L.ptr(pooled2d), _dt(pooled2d),
           pooled2d.stride(0), L.ptr(cache_row0), L.ptr(pool_row0), L.ptr(past), L.ptr(n_new))


ACT_XIELU, ACT_SIGMOID_GATE = 0, 1


def act_rows(x, kind, params=None, gate=None, out_dtype=None):
    """``ACT_XIELU``: z > 0: softplus(p) z^2 + z / 2, z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2 with ``params`` = fp32 [p, q];
    ``ACT_SIGMOID_GATE``: x * sigmoid(gate).  Rows may be views with any pitch."""
    L.require_gpu(x, params, gate)
    _rows(x, "act_rows(x)")
    if kind == ACT_XIELU and (params is None or params.dtype != F32 or params.numel() != 2 or not params.is_contiguous()):
        raise ValueError("act_rows: xIELU takes fp32 [p, q]")
    if kind == ACT_SIGMOID_GATE:
        _rows(gate, "act_rows(gate)")
        if gate.shape != x.shape:
            raise ValueError("act_rows: the gate has x's shape")
    out = torch.empty(x.shape, dtype=out_dtype or x.dtype, device=x.device)
    L.call("mi355_act_rows", x.shape[0], x.shape[1], L.ptr(x), _dt(x), x.stride(0), L.ptr(gate), 0 if gate is None else _dt(gate), 0 if gate is None else gate.stride(0),
           int(kind), L.ptr(params), L.ptr(out), _dt(out), out.stride(0))
    return out


def _vec32(t, n, name):
    if t is not None and (t.dtype != F32 or not t.is_contiguous() or t.numel() != n):
        raise ValueError(f"{name}: contiguous fp32 [{n}] required")


def dyt_sum(x, ya=None, wa=None, ca=1.0, yb=None, wb=None, cb=1.0, y2=None, parts=1, ls=None, eps=0.0, x_out=None, norm=None, out_dtype=None, want32=False):
    """The residual sum of a pre-norm block with statistic-free norms: y = ca N_a(ya) + cb N_b(yb) + (sum of y2's ``parts`` rows per token), N an RMS norm
    over the row with the branch's weight (``wa`` / ``wb`` fp32 [width]) where it has one; v = x + ls * y (``ls`` fp32 [width]: the layer scale).  ``x_out``
    (True: a new tensor, or a tensor, or None) receives v.  ``norm`` = (alpha, weight, bias): tanh(alpha v) weight + bias is returned in ``out_dtype``
    (and as fp32 with ``want32``).  Returns (x_out or None, normed or None, normed fp32 or None)."""
    L.require_gpu(x, ya, wa, yb, wb, y2, ls)
    _rows(x, "dyt_sum(x)")
    T, width = x.shape
    if x.dtype != F32 or not x.is_contiguous():
        raise ValueError("dyt_sum: x contiguous fp32 [tokens, width]")
    for y, n, rows in ((ya, "ya", T), (yb, "yb", T), (y2, "y2", T * parts)):
        if y is not None:
            _rows(y, f"dyt_sum({n})")
            if tuple(y.shape) != (rows, width):
                raise ValueError(f"dyt_sum({n}): [{rows}, {width}] required, got {tuple(y.shape)}")
    for v, n in ((wa, "wa"), (wb, "wb"), (ls, "ls")):
        _vec32(v, width, f"dyt_sum({n})")
    if x_out is True:
        x_out = torch.empty_like(x)
    out = out32 = None
    alpha, w, b = 0.0, None, None
    if norm is not None:
        alpha, w, b = norm
        L.require_gpu(x, w, b)
        _vec32(w, width, "dyt_sum(weight)")
        _vec32(b, width, "dyt_sum(bias)")
        od = out_dtype or F32
        out = torch.empty((T, width), dtype=od, device=x.device)
        out32 = out if od == F32 else (torch.empty((T, width), dtype=F32, device=x.device) if want32 else None)
    L.call("mi355_dyt_sum", T, width, L.ptr(x), L.ptr(ya), 0 if ya is None else _dt(ya), 0 if ya is None else ya.stride(0), L.ptr(wa), float(ca), L.ptr(yb),
           0 if yb is None else _dt(yb), 0 if yb is None else yb.stride(0), L.ptr(wb), float(cb), L.ptr(y2), 0 if y2 is None else _dt(y2), 0 if y2 is None else y2.stride(0),
           int(parts), L.ptr(ls), float(eps), L.ptr(x_out), float(alpha), L.ptr(w), L.ptr(b), L.ptr(out), 0 if out is None else _dt(out), None if out32 is out else L.ptr(out32))
    return x_out, out, out32


def token_shift(h, mu, state, row_seq, seq_off, slot, out_dtype):
    """h fp32 [tokens, C], mu fp32 [n_mix, C] -> [tokens, n_mix * C]: blend s of a row is h + (h' - h) mu[s], h' the sequence's previous row (``state`` fp32
    [slots, C] before the step's first one; read, then set to the step's last row)."""
    L.require_gpu(h, mu, state, row_seq, seq_off, slot)
    _rows(h, "token_shift(h)")
    T, C = h.shape
    n_seq = slot.numel()
    if h.dtype != F32 or mu.dtype != F32 or not mu.is_contiguous() or mu.dim() != 2 or mu.shape[1] != C:
        raise ValueError("token_shift: h fp32 rows, mu contiguous fp32 [n_mix, C]")
    if state.dtype != F32 or not state.is_contiguous() or tuple(state.shape[1:]) != (C,):
        raise ValueError("token_shift: state contiguous fp32 [slots, C]")
    _i32(row_seq, "token_shift(row_seq)", T)
    _i32(seq_off, "token_shift(seq_off)", n_seq + 1)
    _i32(slot, "token_shift(slot)")
    out = torch.empty((T, mu.shape[0] * C), dtype=out_dtype, device=h.device)
    L.call("mi355_token_shift", T, n_seq, C, mu.shape[0], L.ptr(h), h.stride(0), L.ptr(mu), L.ptr(row_seq), L.ptr(seq_off), L.ptr(slot), L.ptr(state), L.ptr(out), _dt(out),
           out.stride(0))
    return out


def _linrec(q, k, v, z, post, u, dt_bias, A_log, D, seq_off, slot, state, H, qk_rep, dk, dv):
    L.require_gpu(q, k, v, z, u, dt_bias, A_log, D, seq_off, slot, state)
    T = q.shape[0]
    G = H // qk_rep
    for t, n, w in ((q, "q", G * dk), (k, "k", G * dk), (v, "v", H * dv), (z, "z", H if post else H * dk)):
        _rows(t, f"linrec({n})")
        if tuple(t.shape) != (T, w):
            raise ValueError(f"linrec({n}): [{T}, {w}] required, got {tuple(t.shape)}")
    if q.dtype != k.dtype or z.dtype != F32:
        raise ValueError("linrec: q / k share a dtype; the decay rows are fp32")
    n_seq = slot.numel()
    _i32(seq_off, "linrec(seq_off)", n_seq + 1)
    _i32(slot, "linrec(slot)")
    if state.dtype != F32 or not state.is_contiguous() or tuple(state.shape[1:]) != (H, dk, dv):
        raise ValueError("linrec: state fp32 [slots, H, dk, dv]")
    o = torch.empty((T, H * dv), dtype=F32, device=q.device)
    L.call("mi355_linrec_ragged", n_seq, L.ptr(seq_off), L.ptr(slot), H, qk_rep, dk, dv, L.ptr(q), L.ptr(k), _dt(q), q.stride(0), k.stride(0), L.ptr(v), _dt(v), v.stride(0),
           L.ptr(z), z.stride(0), 1 if post else 0, L.ptr(u), L.ptr(dt_bias), L.ptr(A_log), L.ptr(D), L.ptr(state), L.ptr(o))
    return o


def decay_bonus_attention(r, k, v, z, u, seq_off, slot, state, H, dk, dv):
    """Linear attention that reads, then updates: o_t = S^T r_t + (sum_i r_i u_i k_i) v_t; S <- diag(exp(-exp(z_t))) S + k_t v_t^T.  z fp32 [tokens, H * dk],
    u fp32 [H * dk], ``state`` fp32 [slots, H, dk, dv].  Returns fp32 [tokens, H * dv]."""
    _vec32(u, H * dk, "decay_bonus_attention(u)")
    return _linrec(r, k, v, z, False, u, None, None, None, seq_off, slot, state, H, 1, dk, dv)


def ssd(c, b, x, dt, dt_bias, A_log, D, seq_off, slot, state, H, G, N, P):
    """State-space duality: per head (group h // (H / G) of b / c) dt = softplus(dt + dt_bias); S <- exp(-exp(A_log) dt) S + b_t (dt x_t)^T;
    y_t = S^T c_t + D x_t.  b, c [tokens, G * N], x [tokens, H * P], dt fp32 [tokens, H]; ``state`` fp32 [slots, H, N, P].  Returns fp32 [tokens, H * P]."""
    for t, n in ((dt_bias, "dt_bias"), (A_log, "A_log"), (D, "D")):
        _vec32(t, H, f"ssd({n})")
    if H % G:
        raise ValueError("ssd: heads must be a multiple of groups")
    return _linrec(c, b, x, dt, True, None, dt_bias, A_log, D, seq_off, slot, state, H, H // G, N, P)


def rglru(u, gates, gbias, lam, y, blocks, seq_off, slot, state, out_dtype, decay_c=8.0):
    """Real-gated linear recurrent unit over a ragged batch: u fp32 [tokens, C], gates fp32 [tokens, 2 C] (per block [recurrence gate | input gate]
    pre-activations, ``gbias`` fp32 [2 C] their biases or None), lam fp32 [C], y [tokens, C] (the GELU branch before its activation); ``state`` fp32 [slots, C].  Returns S * gelu(y)."""
    L.require_gpu(u, gates, gbias, lam, y, seq_off, slot, state)
    for t, n in ((u, "u"), (gates, "gates"), (y, "y")):
        _rows(t, f"rglru({n})")
    T, C = u.shape
    if u.dtype != F32 or gates.dtype != F32 or tuple(gates.shape) != (T, 2 * C) or tuple(y.shape) != (T, C) or C % blocks:
        raise ValueError("rglru: u fp32 [tokens, C], gates fp32 [tokens, 2 C], y [tokens, C], C a multiple of blocks")
    _vec32(lam, C, "rglru(lam)")
    _vec32(gbias, 2 * C, "rglru(gbias)")
    n_seq = slot.numel()
    _i32(seq_off, "rglru(seq_off)", n_seq + 1)
    _i32(slot, "rglru(slot)")
    if state.dtype != F32 or not state.is_contiguous() or tuple(state.shape[1:]) != (C,):
        raise ValueError("rglru: state contiguous fp32 [slots, C]")
    out = torch.empty((T, C), dtype=out_dtype, device=u.device)
    L.call("mi355_rglru_ragged", n_seq, C, int(blocks), float(decay_c), L.ptr(u), u.stride(0), L.ptr(gates), gates.stride(0), L.ptr(gbias), L.ptr(lam), L.ptr(y), _dt(y), y.stride(0),
           L.ptr(seq_off), L.ptr(slot), L.ptr(state), L.ptr(out), _dt(out), out.stride(0))
    return out


def gated_groupnorm(o, w, gate, groups, eps, out_dtype, gate_first=False):
    """o fp32 [tokens, n] in ``groups`` equal consecutive groups, w fp32 [n]: o / rms_group(o) * w * silu(gate), or -- ``gate_first`` -- the RMS norm of
    o * silu(gate) times w."""
    L.require_gpu(o, w, gate)
    _rows(o, "gated_groupnorm(o)")
    _rows(gate, "gated_groupnorm(gate)")
    T, n = o.shape
    if o.dtype != F32 or gate.shape != o.shape or n % groups:
        raise ValueError("gated_groupnorm: o fp32 [tokens, n], gate of that shape, n a multiple of groups")
    _vec32(w, n, "gated_groupnorm(w)")
    out = torch.empty((T, n), dtype=out_dtype, device=o.device)
    L.call("mi355_gated_groupnorm", T, n, int(groups), L.ptr(o), o.stride(0), L.ptr(w), L.ptr(gate), _dt(gate), gate.stride(0), 1 if gate_first else 0, float(eps), L.ptr(out),
           _dt(out), out.stride(0))
    return out


UNARY_RELU2, UNARY_TANH, UNARY_HEAD_GATE = 0, 1, 2


def unary_rows(x, kind, gate=None, group=1, out_dtype=None):
    """``UNARY_RELU2``: relu(x)^2; ``UNARY_TANH``; ``UNARY_HEAD_GATE``: x[r, i] * sigmoid(gate[r, i // group]) (gate [rows, n / group])."""
    L.require_gpu(x, gate)
    _rows(x, "unary_rows(x)")
    if kind == UNARY_HEAD_GATE:
        _rows(gate, "unary_rows(gate)")
        if x.shape[1] % group or tuple(gate.shape) != (x.shape[0], x.shape[1] // group):
            raise ValueError("unary_rows: one gate per run of `group` entries")
    out = torch.empty(x.shape, dtype=out_dtype or x.dtype, device=x.device)
    L.call("mi355_unary_rows", x.shape[0], x.shape[1], L.ptr(x), _dt(x), x.stride(0), int(kind), L.ptr(gate), 0 if gate is None else _dt(gate),
           0 if gate is None else gate.stride(0), int(group), L.ptr(out), _dt(out), out.stride(0))
    return out


def scaled_rope_frequencies(dims, base, scaling, device):
    """fp32 [dims / 2]: base^(-2i / dims), rescaled for a longer context than the one trained on (``scaling`` = {factor, low, high, original}, or None):
    a frequency whose wavelength is shorter than original / high stays, one longer than original / low is divided by factor, between the two the
    frequency is blended linearly in original / wavelength.  Evaluated in double."""
    import math

    i = torch.arange(dims // 2, dtype=torch.float64)
    f = torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / dims)
    if scaling:
        fac, lo, hi, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
        wl = 2.0 * math.pi / f
        smooth = (orig / wl - lo) / (hi - lo) if hi != lo else torch.ones_like(f)
        mid = (1.0 - smooth) * f / fac + smooth * f
        f = torch.where(wl < orig / hi, f, torch.where(wl > orig / lo, f / fac, mid))
    return f.to(F32).to(device)

"""Token mixers and the routed feed-forward of hybrid decoders served in ragged batches, as modules whose constants are constructor arguments:

* ``LatentAttention``       -- multi-head latent attention: queries and keys / values go through low-rank latents, one rotated key part is shared by all
  heads, only the normalised latent and that rotated part are cached (optionally another layer's);
* ``GatedLinearAttention``  -- linear attention with a per-key-channel decay and a matrix state per head, carried in fp32;
* ``GroupedSigmoidMoE``     -- sigmoid-scored experts chosen inside the best groups, squared-ReLU experts;
* ``ShortConvInput``        -- h + conv(h), a short causal convolution over time in front of a mixer, its last inputs carried per sequence;
* ``Retention``             -- linear attention with one fixed decay per head (rotate-half rotary, gated unit-RMS output);
* ``SlidingWindowAttention``-- grouped-query softmax attention with biases, query / key norm, a temperature per head and a window that keeps the first tokens;
* ``GatedDeltaRule``        -- the gated delta rule behind short convolutions, unit-vector queries and keys, a matrix state per value head in fp32;
* ``GatedMLP`` / ``SoftmaxTopkMoE`` -- a dense GELU-gated layer; softmax-routed experts with a clamped gated activation, weights = the winners' scores;
* ``ActMLP``                -- an un-gated feed-forward around the xIELU activation;
* ``SideBySide``            -- two mixers that read the same rows through ONE input product, their outputs joined by the residual kernel (each RMS-normed
  with its own weight, or each with its own factor);
* ``RecurrentGatedUnit``    -- a GELU branch times a real-gated linear recurrent unit behind a short convolution, block-diagonal gates, state in fp32;
* ``StateSpaceDuality``     -- a selective state-space layer with one decay per head and token, a matrix state per head in fp32, gate before a grouped norm;
* ``DecayBonusAttention``   -- token-shifted linear attention with a data-dependent decay per key channel and a bonus for the current token;
* ``Relu2MLP``              -- an un-gated feed-forward around the squared ReLU.
``LatentAttention`` also runs without a query latent, with rotate-half rotary, a sliding window and a sigmoid output gate; ``SlidingWindowAttention`` also
with capped scores, a position-dependent query temperature, pooled blocks before the window, a sink in the denominator, value mixing between layers,
chunks instead of a window, rescaled rotary frequencies and one sigmoid output gate per head; ``SoftmaxTopkMoE`` also with a router bias, weights that are the
softmax over the winners alone, SiLU-gated experts and a shared expert.

They run one *step* of a batch (``SeqStep``): the new tokens of every sequence, packed row after row, against what ``utils.SlotStateCache`` holds.  Inference
only, HIP kernels only (``kernels_seq``); weights are bf16, what is normalised, rotated, decayed, accumulated over time or routed is fp32.
"""

import torch
import torch.nn as nn

from llm_quest_amd import _lib as L
from llm_quest_amd import kernels_seq as S

BF16, F32, I32 = torch.bfloat16, torch.float32, torch.int32


class SeqStep:
    """One step of a ragged batch: ``entries`` = [(slot, new tokens)], the cache gives every sequence's length and last token.  Holds the device-side
    descriptors the kernels read.  ``fresh``: every sequence starts at its first token (prompts; attention may rebuild keys and values from this step's rows)."""

    def __init__(self, cache, entries, device, act_dtype):
        self.cache, self.act_dtype, self.device = cache, act_dtype, device
        import numpy as np

        seq_off, slots, past, n_new = [0], [], [], []
        for slot, new in entries:
            if len(new) == 0:
                raise ValueError("SeqStep: a sequence of the step brings no token")
            seq_off.append(seq_off[-1] + len(new))
            slots.append(slot)
            past.append(cache.length[slot])
            n_new.append(len(new))
        cache.reserve(max(p + n for p, n in zip(past, n_new)))
        cap = cache.capacity
        self.T, self.n_seq, self.max_new = seq_off[-1], len(slots), max(n_new)
        self.max_keys = max(p + n for p, n in zip(past, n_new))
        self.fresh = all(p == 0 for p in past)
        self.host_seq_off, self.host_past, self.host_n_new = seq_off, past, n_new
        T, n = self.T, self.n_seq
        row0 = [s * cap for s in slots]
        # rows of the descriptor block: tokens | previous token | position | cache row | per-sequence arrays | 0 .. T-1 | sequence of a row; one
        # host-to-device copy for all
        buf = np.empty(6 * T + 5 * n + 1, dtype=np.int32)
        tok, prev, pos, dst = buf[0:T], buf[T : 2 * T], buf[2 * T : 3 * T], buf[3 * T : 4 * T]
        for i, (slot, new) in enumerate(entries):
            a, b = seq_off[i], seq_off[i + 1]
            tok[a:b] = new
            prev[a] = cache.last_token[slot]
            prev[a + 1 : b] = tok[a : b - 1]
            pos[a:b] = np.arange(past[i], past[i] + n_new[i], dtype=np.int32)
            dst[a:b] = pos[a:b] + row0[i]
        at = 4 * T
        for arr in (seq_off, slots, past, n_new, row0):
            buf[at : at + len(arr)] = arr
            at += len(arr)
        buf[at : at + T] = np.arange(T, dtype=np.int32)
        buf[at + T : at + 2 * T] = np.repeat(np.arange(n, dtype=np.int32), n_new)
        buf = torch.from_numpy(buf).to(device, non_blocking=False)
        cuts = [T, T, T, T, n + 1, n, n, n, n, T, T]
        parts, at = [], 0
        for c in cuts:
            parts.append(buf[at : at + c])
            at += c
        (self.tok, self.prev, self.pos, self.dst_row, self.seq_off, self.slots, self.past, self.n_new, self.cache_row0, self.local_row, self.row_seq) = parts
        self.q_row0 = self.seq_off[:n]
        self.local = {}  # layer -> this step's latent rows [T, rank + rot] (prompts: the expanded form reads them instead of the cache)
        self.shared = {}  # what one layer leaves for later layers of the same step (the first value-mixing layer's values)
        self._pool_row0 = {}

    def pool_row0(self, blocks_per_slot):
        """int32 [n_seq]: the first pooled row of every sequence in a buffer with ``blocks_per_slot`` rows per slot."""
        if blocks_per_slot not in self._pool_row0:
            self._pool_row0[blocks_per_slot] = (self.slots * blocks_per_slot).to(I32).contiguous()
        return self._pool_row0[blocks_per_slot]

    def completed_blocks(self, pool):
        """The most blocks of ``pool`` positions that one sequence of the step completes."""
        return max((p + n) // pool - p // pool for p, n in zip(self.host_past, self.host_n_new))


def _f32(t):
    return None if t is None else t.detach().to(F32).contiguous()


class _Frozen(nn.Module):
    """Inference-only module: bf16 parameters without gradients; fp32 copies of the small vectors are made once per device (``prepare``)."""

    def _param(self, *shape):
        return nn.Parameter(torch.zeros(*shape, dtype=BF16), requires_grad=False)


class LatentAttention(_Frozen):
    """Multi-head latent attention.  Per head ``dim`` unrotated + ``rot_dim`` rotated query / key entries, ``vdim`` values; latents of ``q_rank`` /
    ``kv_rank``.  ``kv_from``: read that layer's cached rows instead of projecting own ones.  Rotary: ``rot_dims`` of the rotated part turn (base
    ``rot_base``), as interleaved pairs or -- ``rot_layout`` 1 -- entry i with entry i + rot_dims / 2.  ``q_rank`` 0: the query is projected from the
    input directly, without a latent.  ``window`` > 0: position i sees the keys j with 0 <= i - j < window.  ``gate``: the concatenated heads are multiplied
    by the sigmoid of a projection of the mixer's input before the output projection."""

    def __init__(self, width, heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, rot_dims, rot_base, eps, layer_idx, kv_from=None, rot_layout=0, window=0, gate=False):
        super().__init__()
        self.width, self.heads, self.dim, self.rot_dim, self.vdim = width, heads, dim, rot_dim, vdim
        self.q_rank, self.kv_rank, self.scale, self.rot_dims, self.rot_base, self.eps = q_rank, kv_rank, float(scale), rot_dims, float(rot_base), float(eps)
        self.layer_idx, self.kv_from = layer_idx, kv_from
        self.rot_layout, self.window, self.gate = int(rot_layout), int(window), bool(gate)
        if rot_dims % 2 or rot_dims > rot_dim:
            raise ValueError("LatentAttention: the rotated entries are an even number <= rot_dim")
        own = kv_from is None
        # projections of the input side by side -> one product: [query latent, or the queries themselves | kv_rank + rot_dim | gate]
        self.q_cols = q_rank if q_rank else heads * (dim + rot_dim)
        self.kv_cols = kv_rank + rot_dim if own else 0
        self.w_down = self._param(self.q_cols + self.kv_cols + (heads * vdim if gate else 0), width)
        self.q_norm = self._param(q_rank) if q_rank else None
        self.kv_norm = self._param(kv_rank) if own else None
        self.w_uq = self._param(heads * (dim + rot_dim), q_rank) if q_rank else None
        self.w_ukv = self._param(heads * (dim + vdim), kv_rank)  # [key up-projection | value up-projection] rows
        self.w_o = self._param(width, heads * vdim)
        self._ready = None

    def cache_spec(self):
        return ("rows", self.kv_rank + self.rot_dim) if self.kv_from is None else ("shared", self.kv_from)

    def prepare(self, device):
        if self._ready != device:
            self.q_norm32 = _f32(self.q_norm)
            self.kv_norm32 = _f32(self.kv_norm)
            self.freq = S.rope_frequencies(self.rot_dims, self.rot_base, device)
            self._ready = device

    @torch.no_grad()
    def step(self, h, st, out_dtype=None):
        """h [T, width] in the activation dtype -> the mixer's output rows [T, width] (``out_dtype``: of the output projection; default h's)."""
        self.prepare(h.device)
        H, dn, dr, dv, R, Rq = self.heads, self.dim, self.rot_dim, self.vdim, self.kv_rank, self.q_cols
        own = self.kv_from is None
        src = self.layer_idx if own else self.kv_from
        cache2d = st.cache.rows2d(self.layer_idx)
        lay, win = self.rot_layout, self.window
        # without a query latent the projection feeds fp32 work only (rotary, the latent's norm, the gate's sigmoid): it leaves the product as fp32
        down = S.linear(h, self.w_down, out_dtype=None if self.q_rank else F32)
        q = S.linear(S.rmsnorm_rows(down[:, :Rq], self.q_norm32, self.eps), self.w_uq) if self.q_rank else down[:, :Rq]
        kv_src = down[:, Rq : Rq + self.kv_cols]
        if own:
            S.latent_kv_append(kv_src, R, dr, self.kv_norm32, self.eps, st.pos, st.dst_row, self.freq, self.rot_dims, cache2d, layout=lay)
        T = h.shape[0]
        if st.fresh:
            # prompts: keys and values per head rebuilt from this step's latent rows, ordinary head-by-head attention
            if own:
                lat = torch.empty((T, R + dr), dtype=st.act_dtype, device=h.device)
                S.latent_kv_append(kv_src, R, dr, self.kv_norm32, self.eps, st.pos, st.local_row, self.freq, self.rot_dims, lat, layout=lay)
                st.local[src] = lat
            lat = st.local[src]
            kv = S.linear(lat[:, :R], self.w_ukv)  # [T, H*dn | H*dv]
            q32 = torch.empty((T, H * (dn + dr)), dtype=F32, device=h.device)
            S.rope_heads(q, H, dn + dr, dn + dr, 0, q32, dn + dr, 0, dn, self.rot_dims, self.freq, st.pos, layout=lay)
            ctx = torch.empty((T, H * dv), dtype=st.act_dtype, device=h.device)
            S.latent_attn(q32, kv[:, : H * dn], lat[:, R:], kv[:, H * dn :], ctx, H, 1, dn, dr, dv, dn + dr, dn, dv, dv,
                          (st.q_row0, st.n_new, st.past, st.q_row0, st.q_row0, st.q_row0), st.max_new, self.scale, window=win)
        else:
            # continuation: the key up-projection folded onto the query, the value up-projection applied after the attention -- the cache rows are
            # keys and values of every head as they stand
            qf = torch.empty((T, H * (R + dr)), dtype=F32, device=h.device)
            S.bgemm(q, self.w_ukv, qf, T, R, dn, batch=H, lda=q.stride(0), a_bs=dn + dr, sbn=1, sbk=R, b_bs=dn * R, ldc=H * (R + dr), c_bs=R + dr)
            S.rope_heads(q, H, dr, dn + dr, dn, qf, R + dr, R, 0, self.rot_dims, self.freq, st.pos, layout=lay)
            hm = 1
            while hm < min(H, 32):
                hm *= 2
            ol = torch.empty((T, H * R), dtype=st.act_dtype, device=h.device)
            for v0 in range(0, R, 512):  # the attention takes values up to 512 wide: a wider latent goes in parts (the scores are the same every time)
                S.latent_attn(qf, cache2d, cache2d[:, R:], cache2d[:, v0:], ol[:, v0:], H, hm, R, dr, min(512, R - v0), R + dr, 0, 0, R,
                              (st.q_row0, st.n_new, st.past, st.cache_row0, st.cache_row0, st.cache_row0), st.max_new, self.scale, max_keys=st.max_keys, window=win)
            ctx = torch.empty((T, H * dv), dtype=st.act_dtype, device=h.device)
            S.bgemm(ol, self.w_ukv[H * dn :], ctx, T, dv, R, batch=H, lda=H * R, a_bs=R, sbn=R, sbk=1, b_bs=dv * R, ldc=H * dv, c_bs=dv)
        if self.gate:
            ctx = S.act_rows(ctx, S.ACT_SIGMOID_GATE, gate=down[:, Rq + self.kv_cols :])
        return S.linear(ctx, self.w_o, out_dtype=out_dtype)


class GatedLinearAttention(_Frozen):
    """Per head a state S [dim, vdim]: S <- diag(a) S + k v^T, o = S^T q with q scaled by dim^-1/2; a = sigmoid(z)^(1/tau) per key channel, z from a
    low-rank projection with bias.  o is RMS-normed per head (one weight [vdim] for all heads), gated by silu of a projection, and projected out."""

    def __init__(self, width, heads, dim, vdim, decay_rank, tau, eps, layer_idx):
        super().__init__()
        self.width, self.heads, self.dim, self.vdim, self.decay_rank, self.tau, self.eps, self.layer_idx = width, heads, dim, vdim, decay_rank, float(tau), float(eps), layer_idx
        # [q | k | v | gate | decay down-projection] rows -> one product
        self.w_in = self._param(2 * heads * dim + 2 * heads * vdim + decay_rank, width)
        self.w_a2 = self._param(heads * dim, decay_rank)
        self.a2_bias = self._param(heads * dim)
        self.norm = self._param(vdim)
        self.w_o = self._param(width, heads * vdim)
        self._ready = None

    def cache_spec(self):
        return ("state", (self.heads, self.dim, self.vdim))

    def prepare(self, device):
        if self._ready != device:
            self.a2_bias32, self.norm32 = _f32(self.a2_bias), _f32(self.norm)
            self._ready = device

    @torch.no_grad()
    def step(self, h, st):
        self.prepare(h.device)
        H, dk, dv = self.heads, self.dim, self.vdim
        proj = S.linear(h, self.w_in)
        a, b, c = H * dk, 2 * H * dk, 2 * H * dk + H * dv
        z = S.linear(proj[:, c + H * dv :], self.w_a2, out_dtype=F32)
        o = S.gla(proj[:, :a], proj[:, a:b], proj[:, b:c], z, self.a2_bias32, 1.0 / self.tau, dk ** -0.5, st.seq_off, st.slots, st.cache.state(self.layer_idx), H, dk, dv)
        mix = S.gated_headnorm(o, self.norm32, proj[:, c : c + H * dv], H, dv, self.eps, st.act_dtype)
        return S.linear(mix, self.w_o)


class GroupedSigmoidMoE(_Frozen):
    """``experts`` feed-forward experts (down(relu(up x)^2), no biases), ``top`` per token.  Scores sigmoid(router x); the choice adds a per-expert
    correction; experts form ``groups`` runs of neighbours of which the ``keep`` best (by the sum of their two largest choice scores) stay eligible;
    weights are the winners' uncorrected scores, normalised and multiplied by ``scale``.  Returns the experts' weighted outputs as ``top`` fp32 rows per
    token, in descending order of the choice score: the sum is taken by the norm kernel that follows."""

    def __init__(self, width, ff, experts, top, groups, keep, scale, correction=True):
        super().__init__()
        self.width, self.ff, self.experts, self.top, self.groups, self.keep, self.scale = width, ff, experts, top, groups, keep, float(scale)
        self.w_router = self._param(experts, width)
        self.correction = nn.Parameter(torch.zeros(experts, dtype=BF16), requires_grad=False) if correction else None
        self.w_up = self._param(experts, ff, width)
        self.w_down = self._param(experts, width, ff)
        self._ready = None

    def prepare(self, device):
        if self._ready != device:
            self.correction32 = _f32(self.correction)
            self._ready = device

    @torch.no_grad()
    def step(self, x32, h):
        """x32: the fp32 residual rows (the router reads them), h: the same rows in the activation dtype -> fp32 [T * top, width]."""
        self.prepare(h.device)
        T, E, top = h.shape[0], self.experts, self.top
        logits = S.router_logits(x32, self.w_router)
        ids, wts = S.moe_route(logits, self.correction32, top, self.groups, self.keep, self.scale)
        offs, perm = S.moe_dispatch(ids.view(-1), E)
        act = torch.empty((T * top, self.ff), dtype=h.dtype, device=h.device)
        S.bgemm(h, self.w_up, act, T * top, self.ff, self.width, batch=E, sbn=self.width, b_bs=self.ff * self.width, grp_offs=offs, a_rows=perm, a_div=top, epi=1)
        out = torch.empty((T * top, self.width), dtype=F32, device=h.device)
        S.bgemm(act, self.w_down, out, T * top, self.width, self.ff, batch=E, sbn=self.ff, b_bs=self.width * self.ff, grp_offs=offs, c_rows=perm, row_scale=wts.view(-1))
        return out


# ----------------------------------------------------------------------------------------------- mechanisms of parallel-sublayer hybrid decoders
def _largest_pow2_divisor(n, cap=32):
    p = 1
    while p * 2 <= cap and n % (p * 2) == 0:
        p *= 2
    return p


class ShortConvInput(_Frozen):
    """h <- h + conv(h): a causal convolution over time on every channel (``taps`` wide, no bias), added to its input.  The last ``taps - 1`` inputs of
    every sequence are carried as the state ``name`` of the layer."""

    def __init__(self, channels, taps, layer_idx, name="canon"):
        super().__init__()
        self.channels, self.taps, self.layer_idx, self.name = channels, taps, layer_idx, name
        self.weight = self._param(channels, taps)
        self._ready = None

    def state_spec(self):
        return {self.name: (self.taps - 1, self.channels)} if self.taps > 1 else {}

    def prepare(self, device):
        if self._ready != device:
            self.weight32 = _f32(self.weight)
            self._ready = device

    @torch.no_grad()
    def step(self, h32, st, out_dtype):
        """h32: fp32 rows -> h + conv(h) in ``out_dtype`` (one rounding, after the sum)."""
        self.prepare(h32.device)
        state = st.cache.state(self.layer_idx, self.name) if self.taps > 1 else None
        return S.ragged_conv(h32, self.weight32, state, st.row_seq, st.seq_off, st.slots, act=False, residual=True, out_dtype=out_dtype)


class Retention(_Frozen):
    """Linear attention with ONE fixed decay per head and no softmax or denominator: S <- decay_h S + k v^T, o = S^T q, the state carried in fp32.
    Rotary positions on q and k in the rotate-half layout (entry i pairs with i + rot_dims / 2); k is scaled by dim^-1/2 after the rotation; every head's
    output is divided by its root mean square, gated by silu of a projection, and projected out."""

    def __init__(self, width, heads, dim, vdim, decay, rot_dims, rot_base, eps, layer_idx):
        super().__init__()
        if len(decay) != heads:
            raise ValueError(f"Retention: {len(decay)} decays for {heads} heads")
        if rot_dims % 2 or rot_dims > dim:
            raise ValueError("Retention: the rotated entries are an even number <= dim")
        self.width, self.heads, self.dim, self.vdim, self.decay, self.rot_dims, self.rot_base, self.eps, self.layer_idx = width, heads, dim, vdim, [float(d) for d in decay], rot_dims, float(rot_base), float(eps), layer_idx
        self.w_in = self._param(2 * heads * dim + 2 * heads * vdim, width)  # [q | k | v | gate] rows -> one product
        self.w_o = self._param(width, heads * vdim)
        self._ready = None

    def cache_spec(self):
        return {"rows": None, "states": {"S": (self.heads, self.dim, self.vdim)}}

    def prepare(self, device):
        if self._ready != device:
            self.decay32 = torch.tensor(self.decay, dtype=torch.float64).to(F32).to(device)
            self.freq = S.rope_frequencies(self.rot_dims, self.rot_base, device) if self.rot_dims else None
            self.ones = torch.ones(self.vdim, dtype=F32, device=device)
            self._ready = device

    @torch.no_grad()
    def step(self, h, st):
        self.prepare(h.device)
        H, dk, dv = self.heads, self.dim, self.vdim
        proj = S.linear(h, self.w_in, out_dtype=F32)
        a, b, c = H * dk, 2 * H * dk, 2 * H * dk + H * dv
        qk = torch.empty((h.shape[0], b), dtype=F32, device=h.device)
        S.rope_heads(proj, 2 * H, dk, dk, 0, qk, dk, 0, 0, self.rot_dims, self.freq, st.pos, layout=1)  # q and k heads side by side: 2 H heads of dim
        o = S.gla(qk[:, :a], qk[:, a:b], proj[:, b:c], None, None, 1.0, 1.0, st.seq_off, st.slots, st.cache.state(self.layer_idx, "S"), H, dk, dv,
                  head_decay=self.decay32, kscale=dk ** -0.5)
        mix = S.gated_headnorm(o, self.ones, proj[:, c:], H, dv, self.eps, st.act_dtype)
        return S.linear(mix, self.w_o)


class SlidingWindowAttention(_Frozen):
    """Grouped-query softmax attention with optional biases on the four projections, an optional RMS norm (one weight for all heads) on every query and key
    head before a rotary embedding of the first ``rot_dims`` entries, score = q.k * scale * temp[h], and a causal sliding window that also keeps the
    first tokens: position i sees j <= i if i - j < window or j < keep_first (window 0: all of them).  Keys and values are cached token-major,
    [kv_heads x dim | kv_heads x vdim] per row.  Further options, each a constant of its own:
      * ``softcap`` > 0      -- the scaled score passes softcap * tanh(score / softcap);
      * ``q_temp`` (coef, every) -- the query at position p is multiplied by 1 + coef * ln(floor((p + 1) / every) + 1);
      * ``pool`` > 0         -- besides the window, one key and one value for every block of ``pool`` tokens that lies wholly before the window, block b
        being seen from position i iff (b + 1) pool - 1 <= i - window; they are the means of the block's cached keys / values and share the softmax;
      * ``sink``             -- a learned number per head whose exponential joins the softmax denominator (no key, no value, not scaled);
      * ``v_mix`` ("first" / "mix") -- the first such layer of a step leaves its values for the later ones, which cache (1 - lam) v + lam v_first;
      * ``chunk`` > 0        -- instead of a window: positions are cut into chunks of that many from the sequence's first token on, i sees j <= i of its own chunk;
      * ``rot_layout`` 1     -- rotary pairs entry i with entry i + rot_dims / 2 (0: neighbours); ``rot_scaling`` {factor, low, high, original} rescales the
        frequencies for a longer context (``kernels_seq.scaled_rope_frequencies``);
      * ``head_gate``        -- head h's output is multiplied by sigmoid(w_g h)_h, one number per head from the mixer's input, before the output projection
        (its rows follow the value rows in ``w_qkv``);
      * ``o_bias``           -- whether the output projection has a bias (default: as ``bias``).
    ``step(..., proj=rows)``: the caller has already taken the input product (with its biases) -- a mixer beside this one shares it."""

    def __init__(self, width, heads, kv_heads, dim, vdim, scale, window, keep_first, rot_dims, rot_base, eps, layer_idx, qk_norm=True, bias=True, temp=True,
                 softcap=0.0, q_temp=None, pool=0, sink=False, v_mix=None, chunk=0, rot_layout=0, rot_scaling=None, head_gate=False, o_bias=None):
        super().__init__()
        if heads % kv_heads:
            raise ValueError("SlidingWindowAttention: heads must be a multiple of kv_heads")
        if rot_dims % 2 or rot_dims > dim:
            raise ValueError("SlidingWindowAttention: the rotated entries are an even number <= dim")
        if pool and (not window or keep_first):
            raise ValueError("SlidingWindowAttention: pooled blocks lie before a window (and exclude kept first tokens)")
        if v_mix not in (None, "first", "mix"):
            raise ValueError("SlidingWindowAttention: v_mix is None, 'first' or 'mix'")
        if chunk and (window or keep_first or pool):
            raise ValueError("SlidingWindowAttention: chunks stand instead of a window (no kept first tokens, no pooled blocks)")
        self.chunk, self.rot_layout, self.rot_scaling, self.head_gate = int(chunk or 0), int(rot_layout), dict(rot_scaling) if rot_scaling else None, bool(head_gate)
        self.width, self.heads, self.kv_heads, self.dim, self.vdim, self.scale, self.window, self.keep_first = width, heads, kv_heads, dim, vdim, float(scale), int(window), int(keep_first)
        self.rot_dims, self.rot_base, self.eps, self.layer_idx = rot_dims, float(rot_base), float(eps), layer_idx
        self.softcap, self.q_temp, self.pool, self.v_mix = float(softcap or 0.0), (float(q_temp[0]), int(q_temp[1])) if q_temp else None, int(pool or 0), v_mix
        n = (heads + kv_heads) * dim + kv_heads * vdim
        self.qkv_rows = n
        self.w_qkv = self._param(n + (heads if head_gate else 0), width)
        self.b_qkv = self._param(n) if bias else None
        self.q_norm = self._param(dim) if qk_norm else None
        self.k_norm = self._param(dim) if qk_norm else None
        self.temp = self._param(heads) if temp else None
        self.sink = self._param(heads) if sink else None
        self.lam = self._param(1) if v_mix == "mix" else None
        self.w_o = self._param(width, heads * vdim)
        self.b_o = self._param(width) if (bias if o_bias is None else o_bias) else None
        self._ready = None

    # a mixer that shares its input product with a neighbour (``SideBySide``) names the parameter that holds its rows and their biases
    in_weight = "w_qkv"

    def in_bias(self):
        if self.b_qkv is None:
            return None
        b = _f32(self.b_qkv)
        return torch.cat([b, b.new_zeros(self.heads)]) if self.head_gate else b

    def cache_spec(self):
        spec = {"rows": self.kv_heads * (self.dim + self.vdim), "states": {}}
        if self.pool:
            spec["pool"] = self.pool
        return spec

    def prepare(self, device):
        if self._ready != device:
            self.b_qkv32, self.q_norm32, self.k_norm32, self.b_o32, self.sink32 = _f32(self.b_qkv), _f32(self.q_norm), _f32(self.k_norm), _f32(self.b_o), _f32(self.sink)
            t = _f32(self.temp) if self.temp is not None else torch.ones(self.heads, dtype=F32, device=device)
            # the score's factors: folded onto the query, unless the scaled score goes through the cap (then the kernel scales)
            self.qscale = None if self.softcap else (t * self.scale).contiguous()
            if self.softcap and self.temp is not None:
                raise ValueError("SlidingWindowAttention: a per-head temperature and a score cap do not combine")
            self.freq = S.scaled_rope_frequencies(self.rot_dims, self.rot_base, self.rot_scaling, device) if self.rot_dims else None
            self.lam32 = float(self.lam.float().item()) if self.lam is not None else 0.0
            self._ready = device

    @torch.no_grad()
    def step(self, h, st, out_dtype=None, proj=None):
        self.prepare(h.device)
        H, G, d, dv = self.heads, self.kv_heads, self.dim, self.vdim
        L_ = self.layer_idx
        cache2d = st.cache.rows2d(L_)
        bias = self.b_qkv32
        if proj is None:
            proj = S.linear(h, self.w_qkv, out_dtype=F32)
        else:
            bias = None  # the shared product added it
        gate = proj[:, self.qkv_rows :] if self.head_gate else None
        proj = proj[:, : self.qkv_rows]
        vmix = None
        if self.v_mix == "mix":
            vmix = st.shared["v_first"]
            if vmix.shape[1] != G * dv:
                raise ValueError("SlidingWindowAttention: value-mixing layers share one value width")
        elif self.v_mix == "first":
            st.shared["v_first"] = proj[:, (H + G) * d :]  # this step's unmixed values (a view: proj stays alive with it)
        q = S.qkv_rows_append(proj, H, G, d, dv, bias, self.q_norm32, self.k_norm32, self.eps, self.qscale, self.rot_dims, self.rot_layout, self.freq, st.pos, st.dst_row,
                              cache2d, q_temp=self.q_temp, vmix=vmix, lam=self.lam32)
        pooled = row0 = None
        if self.pool:
            p2d = st.cache.pooled2d(L_)
            row0 = st.pool_row0(st.cache.pool_capacity(L_))
            S.pool_rows_update(cache2d, p2d, self.pool, st.cache_row0, row0, st.past, st.n_new, st.completed_blocks(self.pool))
            pooled = (p2d, p2d[:, G * d :])
        ctx = torch.empty((h.shape[0], H * dv), dtype=st.act_dtype, device=h.device)
        hm = _largest_pow2_divisor(H // G)
        S.latent_attn(q, cache2d, None, cache2d[:, G * d :], ctx, H, hm, d, 0, dv, d, d, dv, dv, (st.q_row0, st.n_new, st.past, st.cache_row0, st.cache_row0, st.cache_row0),
                      st.max_new, self.scale if self.softcap else 1.0, max_keys=st.max_keys, kv_rep=H // G, window=self.window, keep_first=self.keep_first,
                      softcap=self.softcap, sink=self.sink32, pool=self.pool, pooled=pooled, pool_row0=row0, chunk=self.chunk)
        if self.head_gate:
            ctx = S.unary_rows(ctx, S.UNARY_HEAD_GATE, gate=gate, group=dv)
        return S.linear(ctx, self.w_o, bias=self.b_o32, out_dtype=out_dtype)


class GatedDeltaRule(_Frozen):
    """Gated delta rule with a matrix state per value head, carried in fp32.  q / k (``kv_heads`` x dim) and v (``heads`` x vdim) pass a short causal
    convolution per channel and silu; q and k become unit vectors per head (q also times dim^-1/2); beta = sigmoid(W_b h); one decay per head,
    g = exp(-exp(A_log) softplus(W_a h + dt_bias)); S <- g S, u = beta (v - S^T k), S <- S + k u^T, o = S^T q.  Every head's output is RMS-normed with
    one weight [vdim], gated by silu of a projection, and projected out."""

    def __init__(self, width, heads, kv_heads, dim, vdim, conv_taps, eps, layer_idx):
        super().__init__()
        if heads % kv_heads:
            raise ValueError("GatedDeltaRule: heads must be a multiple of kv_heads")
        self.width, self.heads, self.kv_heads, self.dim, self.vdim, self.conv_taps, self.eps, self.layer_idx = width, heads, kv_heads, dim, vdim, conv_taps, float(eps), layer_idx
        self.channels = 2 * kv_heads * dim + heads * vdim
        self.w_in = self._param(self.channels + heads * vdim + 2 * heads, width)  # [q | k | v | gate | b | a] rows -> one product
        self.conv = self._param(self.channels, conv_taps)
        self.A_log, self.dt_bias = self._param(heads), self._param(heads)
        self.norm = self._param(vdim)
        self.w_o = self._param(width, heads * vdim)
        self._ready = None

    def cache_spec(self):
        states = {"S": (self.heads, self.dim, self.vdim)}
        if self.conv_taps > 1:
            states["conv"] = (self.conv_taps - 1, self.channels)
        return {"rows": None, "states": states}

    def prepare(self, device):
        if self._ready != device:
            self.conv32, self.A_log32, self.dt_bias32, self.norm32 = _f32(self.conv), _f32(self.A_log), _f32(self.dt_bias), _f32(self.norm)
            self._ready = device

    @torch.no_grad()
    def step(self, h, st):
        self.prepare(h.device)
        H, G, dk, dv, C = self.heads, self.kv_heads, self.dim, self.vdim, self.channels
        proj = S.linear(h, self.w_in, out_dtype=F32)
        state = st.cache.state(self.layer_idx, "conv") if self.conv_taps > 1 else None
        qkv = S.ragged_conv(proj[:, :C], self.conv32, state, st.row_seq, st.seq_off, st.slots, act=True, residual=False, out_dtype=F32)
        a, b = G * dk, 2 * G * dk
        gate0 = C + H * dv
        o = S.delta_rule(qkv[:, :a], qkv[:, a:b], qkv[:, b:], proj[:, gate0 : gate0 + H], proj[:, gate0 + H :], self.A_log32, self.dt_bias32, dk ** -0.5, st.seq_off, st.slots,
                         st.cache.state(self.layer_idx, "S"), H, G, dk, dv)
        mix = S.gated_headnorm(o, self.norm32, proj[:, C:gate0], H, dv, self.eps, st.act_dtype)
        return S.linear(mix, self.w_o)


class GatedMLP(_Frozen):
    """Dense gated feed-forward: down(act(gate x) * (up x)), act = the tanh form of GELU (or ``act`` = ``kernels_seq.GLU_SILU``); gate and up are one product."""

    def __init__(self, width, ff, act=S.GLU_GELU_TANH):
        super().__init__()
        self.width, self.ff, self.act = width, ff, act
        self.w_gate_up = self._param(2 * ff, width)
        self.w_down = self._param(width, ff)
        self.top = 1

    @torch.no_grad()
    def step(self, h32, h, out_dtype=None):
        return S.linear(S.glu_rows(S.linear(h, self.w_gate_up), self.act), self.w_down, out_dtype=out_dtype)


class SoftmaxTopkMoE(_Frozen):
    """``experts`` gated feed-forward experts without biases, ``top`` per token.  Router: fp32 logits, softmax over ALL experts, the ``top`` largest scores
    win and ARE the weights (not renormalised).  Expert: g = min(gate x, limit), u = clamp(up x, -limit, limit), down(g sigmoid(1.702 g) (u + 1)).
    Returns the weighted outputs as ``top`` fp32 rows per token; the sum is taken by the residual kernel that follows.  Options: ``act`` "silu": the expert is
    down(silu(gate x) (up x)); ``router_bias``: a bias on the router's logits; ``chosen_softmax``: the weights are the softmax over the winners' logits alone;
    ``shared_ff`` > 0: a dense expert of the same form (``self.shared``) that every token uses -- ``step`` then returns (expert rows, shared rows [T, width])."""

    def __init__(self, width, ff, experts, top, limit=0.0, act="clamped", router_bias=False, chosen_softmax=False, shared_ff=0):
        super().__init__()
        if act not in ("clamped", "silu"):
            raise ValueError("SoftmaxTopkMoE: act is 'clamped' or 'silu'")
        self.width, self.ff, self.experts, self.top, self.limit = width, ff, experts, top, float(limit)
        self.act, self.chosen_softmax = act, bool(chosen_softmax)
        self.b_router = self._param(experts) if router_bias else None
        if shared_ff and act != "silu":
            raise ValueError("SoftmaxTopkMoE: the shared expert comes with SiLU-gated experts")
        self.shared = GatedMLP(width, shared_ff, act=S.GLU_SILU) if shared_ff else None
        self._ready = None
        self.w_router = self._param(experts, width)
        self.w_gate_up = self._param(experts, 64 * (-(-ff // 32)), width)  # per expert S.pack_gate_up(gate, up): [32 gate rows | 32 up rows] blocks
        self.w_down = self._param(experts, width, ff)

    def load_experts(self, gates, ups, downs):
        """Per-expert weight lists in the checkpoint's layout ([ff, width], [ff, width], [width, ff]) -> the stacked parameters."""
        self.w_gate_up.data.copy_(torch.stack([S.pack_gate_up(g, u) for g, u in zip(gates, ups)]))
        self.w_down.data.copy_(torch.stack(list(downs)))

    @torch.no_grad()
    def step(self, h32, h):
        """h32: the normed fp32 rows (the router reads them), h: the same rows in the activation dtype -> fp32 [T * top, width]."""
        T, E, top, ff = h.shape[0], self.experts, self.top, self.ff
        if self._ready != h.device:
            self.b_router32 = _f32(self.b_router)
            self._ready = h.device
        logits = S.router_logits(h32, self.w_router)
        if self.chosen_softmax:
            ids, wts = S.moe_route(logits, self.b_router32, top, 1, 1, 1.0, softmax="chosen")
        else:
            if self.b_router32 is not None:
                raise ValueError("SoftmaxTopkMoE: a router bias comes with weights over the winners")
            ids, wts = S.moe_route(logits, None, top, 1, 1, 1.0, softmax=True)
        offs, perm = S.moe_dispatch(ids.view(-1), E)
        np_ = self.w_gate_up.shape[1]
        act = torch.empty((T * top, ff), dtype=h.dtype, device=h.device)  # the gated activation is the gate-up product's epilogue
        S.bgemm(h, self.w_gate_up, act, T * top, np_, self.width, batch=E, sbn=self.width, b_bs=np_ * self.width, grp_offs=offs, a_rows=perm, a_div=top,
                epi=S.EPI_SILU_GLU if self.act == "silu" else S.EPI_CLAMPED_SWISH_GLU, limit=self.limit, n_out=ff)
        out = torch.empty((T * top, self.width), dtype=F32, device=h.device)
        S.bgemm(act, self.w_down, out, T * top, self.width, ff, batch=E, sbn=ff, b_bs=self.width * ff, grp_offs=offs, c_rows=perm, row_scale=wts.view(-1))
        if self.shared is not None:
            return out, self.shared.step(h32, h, out_dtype=F32)
        return out


class ActMLP(_Frozen):
    """Un-gated feed-forward: down(act(up x)) with the xIELU activation -- z > 0: softplus(p) z^2 + z / 2; z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2,
    p and q two learned numbers of the layer."""

    def __init__(self, width, ff):
        super().__init__()
        self.width, self.ff = width, ff
        self.w_up = self._param(ff, width)
        self.w_down = self._param(width, ff)
        self.act = self._param(2)
        self._ready = None

    def prepare(self, device):
        if self._ready != device:
            self.act32 = _f32(self.act)
            self._ready = device

    @torch.no_grad()
    def step(self, h, out_dtype=None):
        self.prepare(h.device)
        return S.linear(S.act_rows(S.linear(h, self.w_up), S.ACT_XIELU, params=self.act32), self.w_down, out_dtype=out_dtype)


# ----------------------------------------------------------------------------------------------- mechanisms of decoders with side-by-side branches
class RecurrentGatedUnit(_Frozen):
    """A recurrent block with two branches of ``channels``: y = gelu_tanh(W_y h + b) and u = conv(W_x h + b), a causal convolution per channel with a bias
    and no activation.  u is cut into ``blocks`` equal parts; in part p: r = sigmoid(A_p u_p + a_p), i = sigmoid(B_p u_p + b_p) with square matrices;
    a = exp(-``decay_c`` r softplus(lam)); S <- a S + sqrt(1 - a^2) (i u), S carried per sequence in fp32 from zero; output W_o (S y).  The gates, the decay
    and the recurrence are fp32; the convolution's last inputs are state too."""

    in_weight = "w_in"

    def __init__(self, width, channels, blocks, conv_taps, layer_idx, decay_c=8.0, name="rg"):
        super().__init__()
        if channels % blocks:
            raise ValueError("RecurrentGatedUnit: channels must be a multiple of blocks")
        self.width, self.channels, self.blocks, self.conv_taps, self.layer_idx, self.decay_c, self.name = width, channels, blocks, conv_taps, layer_idx, float(decay_c), name
        n = channels // blocks
        self.w_in = self._param(2 * channels, width)  # [y | x] rows
        self.b_in = self._param(2 * channels)
        self.conv, self.conv_b = self._param(channels, conv_taps), self._param(channels)
        self.w_gates = self._param(blocks, 2 * n, n)  # per block [recurrence-gate rows | input-gate rows]
        self.b_gates = self._param(blocks * 2 * n)
        self.lam = self._param(channels)
        self.w_o = self._param(width, channels)
        self._ready = None

    def load_gates(self, ra, ra_b, ri, ri_b):
        """[blocks, n, n] / [blocks, n] pairs in the checkpoint's layout -> the per-block stacked parameters."""
        self.w_gates.data.copy_(torch.cat([ra, ri], dim=1))
        self.b_gates.data.copy_(torch.cat([ra_b, ri_b], dim=1).reshape(-1))

    def in_bias(self):
        return _f32(self.b_in)

    def cache_spec(self):
        states = {self.name + "_S": (self.channels,)}
        if self.conv_taps > 1:
            states[self.name + "_conv"] = (self.conv_taps - 1, self.channels)
        return {"rows": None, "states": states}

    def prepare(self, device):
        if self._ready != device:
            self.b_in32, self.conv32, self.conv_b32, self.b_gates32, self.lam32 = _f32(self.b_in), _f32(self.conv), _f32(self.conv_b), _f32(self.b_gates), _f32(self.lam)
            self._ready = device

    @torch.no_grad()
    def step(self, h, st, out_dtype=None, proj=None):
        self.prepare(h.device)
        C, nb = self.channels, self.blocks
        n = C // nb
        if proj is None:
            proj = S.linear(h, self.w_in, out_dtype=F32, bias=self.b_in32)
        T = proj.shape[0]
        state = st.cache.state(self.layer_idx, self.name + "_conv") if self.conv_taps > 1 else None
        u = S.ragged_conv(proj[:, C:], self.conv32, state, st.row_seq, st.seq_off, st.slots, act=False, residual=False, out_dtype=F32, bias=self.conv_b32)
        gates = torch.empty((T, 2 * C), dtype=F32, device=h.device)
        S.bgemm(u, self.w_gates, gates, T, 2 * n, n, batch=nb, a_bs=n, sbn=n, b_bs=2 * n * n, c_bs=2 * n)
        mix = S.rglru(u, gates, self.b_gates32, self.lam32, proj[:, :C], nb, st.seq_off, st.slots, st.cache.state(self.layer_idx, self.name + "_S"), st.act_dtype, self.decay_c)
        return S.linear(mix, self.w_o, out_dtype=out_dtype)


class StateSpaceDuality(_Frozen):
    """A selective state-space layer: W_in h = [z: inner | x: inner | B: groups x state | C: groups x state | dt: heads], inner = heads x vdim.  x, B, C pass
    a causal convolution per channel (with bias) and silu; dt = softplus(dt + dt_bias), no clamp.  Per head (group h // (heads / groups)):
    S <- exp(-exp(A_log) dt) S + dt B x^T (S is state x vdim, fp32, from zero), y = S^T C + D x.  y silu(z) is RMS-normed in ``norm_groups`` equal parts,
    times a weight, and projected out: the gate comes before the norm."""

    in_weight = "w_in"

    def __init__(self, width, heads, vdim, state, groups, norm_groups, conv_taps, eps, layer_idx, name="ssd"):
        super().__init__()
        if heads % groups or (heads * vdim) % norm_groups:
            raise ValueError("StateSpaceDuality: heads must be a multiple of groups, heads x vdim of norm_groups")
        self.width, self.heads, self.vdim, self.state, self.groups, self.norm_groups, self.conv_taps, self.eps, self.layer_idx, self.name = (
            width, heads, vdim, state, groups, norm_groups, conv_taps, float(eps), layer_idx, name)
        self.inner = heads * vdim
        self.channels = self.inner + 2 * groups * state
        self.w_in = self._param(self.inner + self.channels + heads, width)
        self.conv, self.conv_b = self._param(self.channels, conv_taps), self._param(self.channels)
        self.dt_bias, self.A_log, self.D = self._param(heads), self._param(heads), self._param(heads)
        self.norm = self._param(self.inner)
        self.w_o = self._param(width, self.inner)
        self._ready = None

    def in_bias(self):
        return None

    def cache_spec(self):
        states = {self.name + "_S": (self.heads, self.state, self.vdim)}
        if self.conv_taps > 1:
            states[self.name + "_conv"] = (self.conv_taps - 1, self.channels)
        return {"rows": None, "states": states}

    def prepare(self, device):
        if self._ready != device:
            self.conv32, self.conv_b32, self.dt_bias32, self.A_log32, self.D32, self.norm32 = (_f32(t) for t in (self.conv, self.conv_b, self.dt_bias, self.A_log, self.D, self.norm))
            self._ready = device

    @torch.no_grad()
    def step(self, h, st, out_dtype=None, proj=None):
        self.prepare(h.device)
        H, P, N, G, I, C = self.heads, self.vdim, self.state, self.groups, self.inner, self.channels
        if proj is None:
            proj = S.linear(h, self.w_in, out_dtype=F32)
        state = st.cache.state(self.layer_idx, self.name + "_conv") if self.conv_taps > 1 else None
        xbc = S.ragged_conv(proj[:, I : I + C], self.conv32, state, st.row_seq, st.seq_off, st.slots, act=True, residual=False, out_dtype=F32, bias=self.conv_b32)
        y = S.ssd(xbc[:, I + G * N :], xbc[:, I : I + G * N], xbc[:, :I], proj[:, I + C :], self.dt_bias32, self.A_log32, self.D32, st.seq_off, st.slots,
                  st.cache.state(self.layer_idx, self.name + "_S"), H, G, N, P)
        mix = S.gated_groupnorm(y, self.norm32, proj[:, :I], self.norm_groups, self.eps, st.act_dtype, gate_first=True)
        return S.linear(mix, self.w_o, out_dtype=out_dtype)


class SideBySide(_Frozen):
    """Two mixers that read the same rows: their input projections are ONE product (the rows of both side by side), each then runs on its part.  The join is
    left to the residual kernel (``kernels_seq.dyt_sum``): ``step`` returns its arguments -- with ``norm_out`` each output is RMS-normed over the width with
    its own plain weight (``left_out`` / ``right_out``) and the two are weighted ``left_scale`` / ``right_scale``; without, just weighted."""

    def __init__(self, left, right, width, left_scale, right_scale, norm_out, eps):
        super().__init__()
        self.left, self.right, self.width, self.left_scale, self.right_scale, self.eps = left, right, width, float(left_scale), float(right_scale), float(eps)
        self.left_out = self._param(width) if norm_out else None
        self.right_out = self._param(width) if norm_out else None
        self._ready = None

    def cache_spec(self):
        a, b = self.left.cache_spec(), self.right.cache_spec()
        if a.get("rows") and b.get("rows"):
            raise ValueError("SideBySide: only one of the two mixers may cache rows")
        spec = {"rows": a.get("rows") or b.get("rows"), "states": {**a["states"], **b["states"]}}
        if len(spec["states"]) != len(a["states"]) + len(b["states"]):
            raise ValueError("SideBySide: the two mixers' states need different names")
        for k in ("pool",):
            if a.get(k) or b.get(k):
                spec[k] = a.get(k) or b.get(k)
        return spec

    def prepare(self, device):
        if self._ready != device:
            wl, wr = getattr(self.left, self.left.in_weight), getattr(self.right, self.right.in_weight)
            self.split = wl.shape[0]
            both = torch.cat([wl.data, wr.data]).contiguous()  # the two input projections side by side; the mixers' own parameters become views of it
            wl.data, wr.data = both[: self.split], both[self.split :]
            self.w_both = both
            bl, br = self.left.in_bias(), self.right.in_bias()
            self.b_both = None
            if bl is not None or br is not None:
                z = lambda n: torch.zeros(n, dtype=F32, device=device)
                self.b_both = torch.cat([bl if bl is not None else z(self.split), br if br is not None else z(wr.shape[0])]).contiguous()
            self.left_out32, self.right_out32 = _f32(self.left_out), _f32(self.right_out)
            self._ready = device

    @torch.no_grad()
    def step(self, h, st):
        self.prepare(h.device)
        proj = S.linear(h, self.w_both, out_dtype=F32, bias=self.b_both)
        ya = self.left.step(h, st, out_dtype=F32, proj=proj[:, : self.split])
        yb = self.right.step(h, st, out_dtype=F32, proj=proj[:, self.split :])
        return dict(ya=ya, wa=self.left_out32, ca=self.left_scale, yb=yb, wb=self.right_out32, cb=self.right_scale, eps=self.eps)


class DecayBonusAttention(_Frozen):
    """Token-shifted linear attention with a matrix state per head (``dim`` x ``dim``, fp32, from zero).  With h' the previous token's input (zeros at the
    start; carried as state), five blends h + (h' - h) mu_s feed r, k, v, the gate and the decay: r, k, v = W_s blend_s, gate = silu(W_g blend_g),
    decay w = exp(-exp(w0 + W_2 tanh(W_1 blend_w))) per head and key channel.  o_t = (S + diag(u) k_t v_t^T)^T r_t -- the bonus u counts for the current
    token only -- then S <- diag(w_t) S + k_t v_t^T.  Every head's o is divided by its root mean square, times a weight over all heads, times the gate,
    and projected out."""

    def __init__(self, width, heads, dim, decay_rank, eps, layer_idx):
        super().__init__()
        self.width, self.heads, self.dim, self.decay_rank, self.eps, self.layer_idx = width, heads, dim, decay_rank, float(eps), layer_idx
        n = heads * dim
        self.mu = self._param(5, width)  # blends of r, k, v, gate, decay
        self.w_rkvg = self._param(4, n, width)
        self.w1, self.w2, self.w0 = self._param(decay_rank, width), self._param(n, decay_rank), self._param(n)
        self.u, self.norm = self._param(n), self._param(n)
        self.w_o = self._param(width, n)
        self._ready = None

    def cache_spec(self):
        return {"rows": None, "states": {"shift": (self.width,), "S": (self.heads, self.dim, self.dim)}}

    def prepare(self, device):
        if self._ready != device:
            self.mu32, self.w0_32, self.u32, self.norm32 = _f32(self.mu), _f32(self.w0), _f32(self.u), _f32(self.norm)
            self._ready = device

    @torch.no_grad()
    def step(self, h32, st, out_dtype=None):
        """h32: the normed rows in fp32 (the blends are taken in fp32 and rounded once)."""
        self.prepare(h32.device)
        H, d, W = self.heads, self.dim, self.width
        n, T = H * d, h32.shape[0]
        mixes = S.token_shift(h32, self.mu32, st.cache.state(self.layer_idx, "shift"), st.row_seq, st.seq_off, st.slots, st.act_dtype)
        rkvg = torch.empty((T, 4 * n), dtype=F32, device=h32.device)
        S.bgemm(mixes, self.w_rkvg, rkvg, T, n, W, batch=4, a_bs=W, sbn=W, b_bs=n * W, c_bs=n)
        lora = S.unary_rows(S.linear(mixes[:, 4 * W :], self.w1, out_dtype=F32), S.UNARY_TANH)
        z = torch.empty((T, n), dtype=F32, device=h32.device)
        S.bgemm(lora, self.w2, z, T, n, self.decay_rank, bias=self.w0_32)
        o = S.decay_bonus_attention(rkvg[:, :n], rkvg[:, n : 2 * n], rkvg[:, 2 * n : 3 * n], z, self.u32, st.seq_off, st.slots, st.cache.state(self.layer_idx, "S"), H, d, d)
        mix = S.gated_groupnorm(o, self.norm32, rkvg[:, 3 * n :], H, self.eps, st.act_dtype, gate_first=False)
        return S.linear(mix, self.w_o, out_dtype=out_dtype)


class Relu2MLP(_Frozen):
    """Un-gated feed-forward: down(relu(up x)^2)."""

    def __init__(self, width, ff):
        super().__init__()
        self.width, self.ff = width, ff
        self.w_up = self._param(ff, width)
        self.w_down = self._param(width, ff)

    @torch.no_grad()
    def step(self, h, out_dtype=None):
        return S.linear(S.unary_rows(S.linear(h, self.w_up), S.UNARY_RELU2), self.w_down, out_dtype=out_dtype)

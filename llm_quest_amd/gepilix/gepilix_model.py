"""Gepilix: a pre-norm decoder whose norms take no statistics -- Dynamic Tanh, tanh(alpha x) w + b -- and whose sublayer outputs pass a per-channel layer
scale: x <- x + s1 * mixer(n1(x)), then x <- x + s2 * ff(n2(x)).  A configurable list of layers whose mixer is
  * *parallel*   -- chunked grouped-query attention (biases, no rotation, capped scores, one sigmoid gate per head) beside a real-gated linear recurrent
    unit; the two outputs are RMS-normed over the width with their own weights and averaged;
  * *parallel_2* -- sliding-window grouped-query attention (rotate-half rotary with rescaled frequencies, capped scores) beside a state-space-duality
    layer; a weighted sum of the two;
  * *wkv*        -- token-shifted linear attention with a data-dependent decay and a bonus for the current token.
The feed-forward is down(relu(up x)^2), a mixture of SiLU-gated experts (top-k by logit, weights = softmax over the winners) plus a shared expert, or
absent.  A final norm and an untied head.  The mechanisms are those of ``common/mixers.py`` (``SideBySide``, ``SlidingWindowAttention``,
``RecurrentGatedUnit``, ``StateSpaceDuality``, ``DecayBonusAttention``, ``Relu2MLP``, ``SoftmaxTopkMoE``) with this design's constants.

Every size and constant comes from the checkpoint's ``config.json`` (``GepilixConfig``) or a tensor's shape; nothing here depends on a particular model
of the design.  Inference only: ``step`` runs one step of a ragged batch against a ``SlotStateCache`` (``generate.RaggedBatch`` drives it).  ``act_dtype``
bf16 is the serving mode (bf16 operands of the matrix products, fp32 accumulation); fp32 runs every product as fp32 FMAs.  In both modes the residual
stream, the norms, rotary angles, attention scores, routers, decays, gates of a recurrence and recurrent state are fp32.
"""

import torch
import torch.nn as nn

from llm_quest_amd import kernels_seq as S
from llm_quest_amd.common.mixers import (DecayBonusAttention, RecurrentGatedUnit, Relu2MLP, SideBySide, SlidingWindowAttention, SoftmaxTopkMoE, StateSpaceDuality, _f32)
from llm_quest_amd.utils import SlotStateCache

BF16, F32 = torch.bfloat16, torch.float32

MIXER_TYPES = ("parallel", "parallel_2", "wkv")
RGLRU_DECAY = 8.0  # the recurrent unit's decay is exp(-8 r softplus(lam))


class GepilixConfig:
    """The parsed ``config.json`` of a Gepilix checkpoint.  ``decay_ranks``: per *wkv* layer the rank of its decay's low-rank projection (a tensor's shape
    gives it; the loader fills it in)."""

    def __init__(self, cfg, decay_ranks=None):
        if cfg.get("architecture") != "Gepilix":
            raise ValueError(f"not a Gepilix config: architecture = {cfg.get('architecture')!r}")
        self.raw = cfg
        self.vocab, self.width = int(cfg["vocab"]), int(cfg["width"])
        self.eps = float(cfg["norm"]["eps"])
        self.layers = cfg["layers"]
        self.context_length = int(cfg.get("context_length", 1 << 20))
        self.decay_ranks = dict(decay_ranks or {})
        for i, layer in enumerate(self.layers):
            if layer["type"] not in MIXER_TYPES:
                raise ValueError(f"layer {i}: unknown mixer type {layer['type']!r}")
            mlp = layer.get("mlp")
            if mlp is not None and mlp.get("kind") not in ("dense", "moe"):
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
            if layer["type"] == "wkv" and i not in self.decay_ranks:
                self.decay_ranks[i] = int(layer["mixer"].get("decay_rank", 16))


def _attention(cfg, m, i, chunked, bias, head_gate):
    mask, rot = m.get("mask") or {}, m.get("rot") or {}
    size = int(mask.get("size", 0))
    return SlidingWindowAttention(cfg.width, m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"], m.get("scale", m["dim"] ** -0.5), 0 if chunked else size, 0,
                                  int(rot.get("dims", 0)), rot.get("base", 10000.0), cfg.eps, i, qk_norm=False, bias=bias, temp=False, softcap=m.get("softcap", 0.0),
                                  chunk=size if chunked else 0, rot_layout=1, rot_scaling=rot.get("scaling"), head_gate=head_gate, o_bias=False)


def _mixer(cfg, i):
    layer, w = cfg.layers[i], cfg.width
    m = layer["mixer"]
    if layer["type"] == "wkv":
        return DecayBonusAttention(w, m["heads"], m["dim"], cfg.decay_ranks[i], cfg.eps, i)
    L, R = m["left"], m["right"]
    if layer["type"] == "parallel":
        left = _attention(cfg, L, i, chunked=True, bias=True, head_gate=True)
        right = RecurrentGatedUnit(w, R["width"], R["blocks"], R.get("conv", 1), i, decay_c=RGLRU_DECAY)
        return SideBySide(left, right, w, 0.5, 0.5, True, cfg.eps)
    left = _attention(cfg, L, i, chunked=False, bias=False, head_gate=False)
    right = StateSpaceDuality(w, R["heads"], R["vdim"], R["state"], R.get("groups", 1), R.get("norm_groups", 1), R.get("conv", 1), cfg.eps, i)
    return SideBySide(left, right, w, m.get("left_scale", 1.0), m.get("right_scale", 1.0), False, cfg.eps)


class DynamicTanh(nn.Module):
    """tanh(alpha x) w + b: a scalar, a weight and a bias; no mean, no variance."""

    def __init__(self, width):
        super().__init__()
        self.alpha = nn.Parameter(torch.ones((), dtype=BF16), requires_grad=False)
        self.weight = nn.Parameter(torch.ones(width, dtype=BF16), requires_grad=False)
        self.bias = nn.Parameter(torch.zeros(width, dtype=BF16), requires_grad=False)

    def triple(self):
        return float(self.alpha.float().item()), _f32(self.weight), _f32(self.bias)


class GepilixBlock(nn.Module):
    def __init__(self, cfg, i):
        super().__init__()
        w = cfg.width
        self.norm1 = DynamicTanh(w)
        self.ls1 = nn.Parameter(torch.ones(w, dtype=BF16), requires_grad=False)
        self.mixer = _mixer(cfg, i)
        mlp = cfg.layers[i].get("mlp")
        self.ff = None
        if mlp is not None:
            self.norm2 = DynamicTanh(w)
            self.ls2 = nn.Parameter(torch.ones(w, dtype=BF16), requires_grad=False)
            if mlp["kind"] == "dense":
                self.ff = Relu2MLP(w, mlp["ff"])
            else:
                shared = mlp.get("shared") or {}
                self.ff = SoftmaxTopkMoE(w, mlp["expert"]["ff"], mlp["router"]["experts"], mlp["router"]["top"], act="silu", router_bias=True, chosen_softmax=True,
                                         shared_ff=int(shared.get("ff", 0)))

    def cache_spec(self):
        return self.mixer.cache_spec()


class GepilixModel(nn.Module):
    def __init__(self, cfg, act_dtype=BF16):
        super().__init__()
        if act_dtype not in (BF16, F32):
            raise TypeError("Gepilix runs with bf16 or fp32 activations")
        self.cfg, self.act_dtype = cfg, act_dtype
        self.embed = nn.Parameter(torch.zeros(cfg.vocab, cfg.width, dtype=BF16), requires_grad=False)
        self.blocks = nn.ModuleList([GepilixBlock(cfg, i) for i in range(len(cfg.layers))])
        self.final_norm = DynamicTanh(cfg.width)
        self.head = nn.Parameter(torch.zeros(cfg.vocab, cfg.width, dtype=BF16), requires_grad=False)
        self._norms = None

    @property
    def vocab_size(self):
        return self.cfg.vocab

    def new_cache(self, device, max_tokens=0, slots=4):
        return SlotStateCache([blk.cache_spec() for blk in self.blocks], self.cfg.context_length, device, self.act_dtype, slots=slots, capacity=max_tokens)

    def _prepare(self):
        if self._norms is None or self._norms[0] != self.embed.device:
            n = [(b.norm1.triple(), _f32(b.ls1), b.norm2.triple() if b.ff is not None else None, _f32(b.ls2) if b.ff is not None else None) for b in self.blocks]
            self._norms = (self.embed.device, n, self.final_norm.triple())
        return self._norms

    @torch.no_grad()
    def step(self, st, want_rows=None, return_layers=False):
        """One step of a ragged batch ``st`` (``SeqStep``).  Returns fp32 logits for the rows ``want_rows`` (int64 device tensor; default: each sequence's
        last row) -- and with ``return_layers`` also the fp32 residual stream after every layer."""
        cfg, act = self.cfg, self.act_dtype
        _, norms, fn = self._prepare()
        x = S.embed_hash(st.tok, st.prev, self.embed, 1.0)
        layers = []
        # a sublayer's output joins the stream (layer scale, branch norms and factors, expert rows) in the kernel that also norms the sum for the next sublayer
        pend = None
        for blk, (n1, ls1, n2, ls2) in zip(self.blocks, norms):
            wkv = isinstance(blk.mixer, DecayBonusAttention)
            x_new, h, _ = S.dyt_sum(x, x_out=None if pend is None else True, norm=n1, out_dtype=F32 if wkv else act, **(pend or {}))
            if pend is not None:
                x = x_new
                if return_layers:
                    layers.append(x)
            if wkv:
                pend = dict(ya=blk.mixer.step(h, st, out_dtype=F32), ls=ls1)
            else:
                pend = dict(blk.mixer.step(h, st), ls=ls1)
            if blk.ff is None:
                continue
            moe = isinstance(blk.ff, SoftmaxTopkMoE)
            x, h, h32 = S.dyt_sum(x, x_out=True, norm=n2, out_dtype=act, want32=moe, **pend)
            if moe:
                out = blk.ff.step(h32, h)
                rows, shared = out if isinstance(out, tuple) else (out, None)
                pend = dict(ya=shared, y2=rows, parts=blk.ff.top, ls=ls2)
            else:
                pend = dict(ya=blk.ff.step(h, out_dtype=F32), ls=ls2)
        x, _, _ = S.dyt_sum(x, x_out=True, **(pend or {}))
        if return_layers:
            layers.append(x)
        if want_rows is None:
            want_rows = (st.seq_off[1:] - 1).long()
        _, hn, _ = S.dyt_sum(x.index_select(0, want_rows), norm=fn, out_dtype=act)
        logits = S.linear(hn, self.head, out_dtype=F32)
        return (logits, layers) if return_layers else logits

"""Mopalorn: a decoder with SANDWICH norms -- x <- x + n1b(mixer(n1(x))), then x <- x + n2b(ff(n2(x))), every norm a plain RMS norm with a weight.  A
configurable list of layers whose mixer is *latent_attention* (keys and values rebuilt from a cached latent, a rotated key part shared by the heads,
rotate-half rotary, a sliding window, a sigmoid output gate), *attention* (grouped queries, no rotation, a query temperature that grows with the logarithm
of the position, tanh-capped scores, every earlier key visible) or *attention_2* (grouped queries, a sliding window plus one mean key / value per block of
tokens that lies wholly before it, a sink in the softmax denominator); layers marked ``v_mix`` blend their values with those of the first such layer.  The
feed-forward is down(xIELU(up x)) or absent.  The head is the embedding table, the logits times a constant.  The mechanisms are those of
``common/mixers.py`` (``LatentAttention``, ``SlidingWindowAttention``, ``ActMLP``) with this design's constants.

Every size and constant comes from the checkpoint's ``config.json`` (``MopalornConfig``); nothing here depends on a particular model of the design.
Inference only: ``step`` runs one step of a ragged batch against a ``SlotStateCache`` (``generate.RaggedBatch`` drives it).  ``act_dtype`` bf16 is the
serving mode (bf16 operands of the matrix products, fp32 accumulation); fp32 runs every product as fp32 FMAs.  In both modes the residual stream, the
norms, rotary angles, the query temperature, attention scores and softmax are fp32.
"""

import torch
import torch.nn as nn

from llm_quest_amd import kernels_seq as S
from llm_quest_amd.common.mixers import ActMLP, LatentAttention, SlidingWindowAttention, _f32
from llm_quest_amd.utils import SlotStateCache

BF16, F32 = torch.bfloat16, torch.float32

MIXER_TYPES = ("latent_attention", "attention", "attention_2")


class MopalornConfig:
    """The parsed ``config.json`` of a Mopalorn checkpoint."""

    def __init__(self, cfg):
        if cfg.get("architecture") != "Mopalorn":
            raise ValueError(f"not a Mopalorn config: architecture = {cfg.get('architecture')!r}")
        self.raw = cfg
        self.vocab, self.width = int(cfg["vocab"]), int(cfg["width"])
        self.eps = float(cfg["norm"]["eps"])
        self.logit_scale = float(cfg.get("logit_scale", 1.0))
        self.layers = cfg["layers"]
        self.context_length = int(cfg.get("context_length", 1 << 20))
        first_mix = None
        self.v_mix = []  # per layer: None, "first" (the first layer that mixes: it only lends its values) or "mix"
        for i, layer in enumerate(self.layers):
            if layer["type"] not in MIXER_TYPES:
                raise ValueError(f"layer {i}: unknown mixer type {layer['type']!r}")
            mlp = layer.get("mlp")
            if mlp is not None and mlp.get("kind") != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
            m = layer["mixer"]
            mixes = layer["type"] != "latent_attention" and bool(m.get("v_mix"))
            if mixes:
                rows = int(m.get("kv_heads", m["heads"])) * int(m["vdim"])
                if first_mix is None:
                    first_mix = rows
                elif rows != first_mix:
                    raise ValueError(f"layer {i}: value mixing needs the value rows of the first mixing layer ({first_mix} wide), got {rows}")
            self.v_mix.append(None if not mixes else ("first" if sum(v is not None for v in self.v_mix) == 0 else "mix"))


def _mixer(cfg, i, has_sink):
    layer, w = cfg.layers[i], cfg.width
    m = layer["mixer"]
    mask = m.get("mask") or {}
    if layer["type"] == "latent_attention":
        rot = m.get("rot") or {"dims": m["rot_dim"], "base": 10000.0}
        return LatentAttention(w, m["heads"], m["dim"], m["rot_dim"], m["vdim"], 0, m["kv_rank"], m.get("scale", (m["dim"] + m["rot_dim"]) ** -0.5), rot["dims"], rot["base"],
                               cfg.eps, i, rot_layout=1, window=mask.get("size", 0), gate=True)
    kw = dict(qk_norm=False, bias=False, temp=False, v_mix=cfg.v_mix[i])
    if layer["type"] == "attention":
        qt = m.get("q_temp")
        kw.update(softcap=m.get("softcap", 0.0), q_temp=(qt["coef"], qt["every"]) if qt else None)
        window = 0
    else:
        kw.update(pool=mask.get("pool", 0), sink=has_sink)
        window = mask.get("size", 0)
    return SlidingWindowAttention(w, m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"], m.get("scale", m["dim"] ** -0.5), window, 0, 0, 10000.0, cfg.eps, i, **kw)


class MopalornBlock(nn.Module):
    def __init__(self, cfg, i, has_sink):
        super().__init__()
        w = cfg.width
        self.norm1, self.norm1b = (nn.Parameter(torch.ones(w, dtype=BF16), requires_grad=False) for _ in range(2))
        self.mixer = _mixer(cfg, i, has_sink)
        mlp = cfg.layers[i].get("mlp")
        self.ff = None
        if mlp is not None:
            self.norm2, self.norm2b = (nn.Parameter(torch.ones(w, dtype=BF16), requires_grad=False) for _ in range(2))
            self.ff = ActMLP(w, mlp["ff"])

    def cache_spec(self):
        return self.mixer.cache_spec()


class MopalornModel(nn.Module):
    """``sinks``: the layers of type ``attention_2`` whose checkpoint holds a sink (default: all of them)."""

    def __init__(self, cfg, act_dtype=BF16, sinks=None):
        super().__init__()
        if act_dtype not in (BF16, F32):
            raise TypeError("Mopalorn runs with bf16 or fp32 activations")
        self.cfg, self.act_dtype = cfg, act_dtype
        self.embed = nn.Parameter(torch.zeros(cfg.vocab, cfg.width, dtype=BF16), requires_grad=False)
        n = len(cfg.layers)
        self.blocks = nn.ModuleList([MopalornBlock(cfg, i, cfg.layers[i]["type"] == "attention_2" and (sinks is None or i in sinks)) for i in range(n)])
        self.final_norm = nn.Parameter(torch.ones(cfg.width, dtype=BF16), requires_grad=False)
        self._norms = None

    @property
    def vocab_size(self):
        return self.cfg.vocab

    def new_cache(self, device, max_tokens=0, slots=4):
        return SlotStateCache([blk.cache_spec() for blk in self.blocks], self.cfg.context_length, device, self.act_dtype, slots=slots, capacity=max_tokens)

    def _prepare(self):
        if self._norms is None or self._norms[0] != self.embed.device:
            n = [(_f32(b.norm1), _f32(b.norm1b), _f32(b.norm2) if b.ff is not None else None, _f32(b.norm2b) if b.ff is not None else None) for b in self.blocks]
            # the constant on the logits rides on the final norm's weight (fp32)
            self._norms = (self.embed.device, n, (_f32(self.final_norm) * self.cfg.logit_scale).contiguous())
        return self._norms

    @torch.no_grad()
    def step(self, st, want_rows=None, return_layers=False):
        """One step of a ragged batch ``st`` (``SeqStep``).  Returns fp32 logits for the rows ``want_rows`` (int64 device tensor; default: each sequence's
        last row) -- and with ``return_layers`` also the fp32 residual stream after every layer."""
        cfg, act = self.cfg, self.act_dtype
        _, norms, fw = self._prepare()
        x = S.embed_hash(st.tok, st.prev, self.embed, 1.0)
        layers = []
        # a sublayer's output meets the stream in the kernel that norms it, adds it, and norms the sum for the next sublayer
        y = post = None
        for blk, (n1, n1b, n2, n2b) in zip(self.blocks, norms):
            x_new, h = S.sandwich_rmsnorm(x, cfg.eps, y=y, w_post=post, w_next=n1, out_dtype=act, x_out=None if y is None else True)
            if y is not None:
                x = x_new
                if return_layers:
                    layers.append(x)
            y, post = blk.mixer.step(h, st, out_dtype=F32), n1b
            if blk.ff is not None:
                x, h = S.sandwich_rmsnorm(x, cfg.eps, y=y, w_post=post, w_next=n2, out_dtype=act, x_out=True)
                y, post = blk.ff.step(h, out_dtype=F32), n2b
        x, _ = S.sandwich_rmsnorm(x, cfg.eps, y=y, w_post=post, x_out=True)
        if return_layers:
            layers.append(x)
        if want_rows is None:
            want_rows = (st.seq_off[1:] - 1).long()
        _, hn = S.sandwich_rmsnorm(x.index_select(0, want_rows), cfg.eps, w_next=fw, out_dtype=act)
        logits = S.linear(hn, self.embed, out_dtype=F32)
        return (logits, layers) if return_layers else logits

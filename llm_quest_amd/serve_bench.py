"""Serving throughput of the registry models with random weights: prompts (one packed step) and one-token steps through the slot cache, beside the
closest existing model of the package at equal width and depth -- the Qwen3.5 hybrid text stack (gated delta net + gated attention, dense SwiGLU) through
its own cache.  ``bench.py --serve gemepel`` (or ``--serve mepatar``) prints the result as one JSON line; the default workload of ``bench.py`` is untouched.
``--serve mopalorn`` stands beside a Mepatar stack of sliding-window attention layers with dense feed-forwards at equal width, depth, heads and parameter
count: the package's closest model to an all-attention decoder with dense layers.  ``--serve gepilix`` stands beside the Mepatar hybrid (recurrent mixers
with a matrix state per head, one windowed attention layer, routed experts) at equal width, depth, heads and expert sizes.

Sizes resemble real layers (random weights; what is generated means nothing): width 1024 / 2048, 4 layers (three linear-attention layers and one softmax-
attention layer, as the Qwen3.5 stack has them), 16 experts of which 2 run per token."""

import json
import time

import torch

BF16 = torch.bfloat16


def gemepel_config(width, heads, vocab=32000):
    lat = {"heads": heads, "dim": 128, "rot_dim": 64, "vdim": 128, "q_rank": width // 2, "kv_rank": 256, "rot": {"dims": 64, "base": 1e6}, "scale": 192 ** -0.5}
    gla = {"heads": 16, "dim": 128, "vdim": 128, "tau": 16.0}
    mlp = {"kind": "moe", "expert": {"ff": int(width * 1.75)}, "router": {"experts": 16, "top": 2, "groups": {"count": 4, "keep": 2}, "scale": 2.5}}
    layers = [{"type": "gla", "mixer": gla, "mlp": mlp}, {"type": "gla", "mixer": gla, "mlp": mlp}, {"type": "gla", "mixer": gla, "mlp": mlp},
              {"type": "latent_attention", "mixer": lat, "mlp": mlp}]
    return {"architecture": "Gemepel", "vocab": vocab, "width": width, "norm": {"eps": 1e-6}, "postln_alpha": 1.0,
            "embedding": {"scale": 1.0, "bigram": {"buckets": 65521, "mul_prev": 31, "mul_cur": 7}}, "layers": layers}


def random_gemepel(width, heads, device, decay_rank=64):
    from llm_quest_amd.gemepel.gemepel_model import GemepelConfig, GemepelModel

    cfg = GemepelConfig(gemepel_config(width, heads))
    shapes = {f"l{i}.mix.a1": (decay_rank, width) for i in range(len(cfg.layers))}
    shapes.update({f"l{i}.mlp.correction": (16,) for i in range(len(cfg.layers))})
    with torch.device(device):
        model = GemepelModel(cfg, shapes)
    g = torch.Generator(device=device).manual_seed(7)
    for name, p in model.named_parameters():
        if p.dim() >= 2:
            p.data.copy_((torch.randn(p.shape, device=device, generator=g) / p.shape[-1] ** 0.5).to(BF16))
        elif name.endswith("_w") or name.endswith("norm"):
            p.data.fill_(1.0)
        elif name.endswith("a2_bias"):
            p.data.fill_(3.0)
    return model


def mepatar_config(width, heads, vocab=32000):
    """Two gated-delta-rule layers, one retention layer and one sliding-window attention layer (512 keys + 4 kept), 16 heads x 128 x 128 in the recurrent
    mixers; three layers with 16 experts (2 per token, ff = 1.75 width) and one dense layer (ff = 3.5 width); 4 taps, norms in 4 groups."""
    rec = {"heads": 16, "dim": 128, "vdim": 128}
    ret = dict(rec, decay=[1.0 - 2.0 ** (-5 - 0.25 * i) for i in range(16)], rot={"dims": 128, "base": 1e6})
    dlt = dict(rec, kv_heads=16, conv=4)
    att = {"heads": heads, "kv_heads": 2, "dim": 128, "vdim": 128, "mask": {"size": 512, "keep_first": 4}, "rot": {"dims": 64, "base": 1e6}, "scale": 128 ** -0.5}
    moe = {"kind": "moe", "expert": {"ff": int(width * 1.75), "limit": 7.0}, "router": {"experts": 16, "top": 2}}
    dense = {"kind": "dense", "ff": int(width * 3.5)}
    layers = [{"type": "delta", "mixer": dlt, "mlp": moe}, {"type": "retention", "mixer": ret, "mlp": dense}, {"type": "delta", "mixer": dlt, "mlp": moe},
              {"type": "attention", "mixer": att, "mlp": moe}]
    return {"architecture": "Mepatar", "vocab": vocab, "width": width, "norm": {"eps": 1e-6, "groups": 4}, "canon": {"taps": 4}, "embedding": {"scale": 1.0}, "layers": layers}


def random_mepatar(width, heads, device):
    from llm_quest_amd.mepatar.mepatar_model import MepatarConfig, MepatarModel

    with torch.device(device):
        model = MepatarModel(MepatarConfig(mepatar_config(width, heads)))
    g = torch.Generator(device=device).manual_seed(7)
    for name, p in model.named_parameters():
        if name.endswith("canon.weight") or name.endswith("mixer.conv"):
            p.data.copy_((0.3 * torch.randn(p.shape, device=device, generator=g)).to(BF16))
        elif p.dim() >= 2:
            p.data.copy_((torch.randn(p.shape, device=device, generator=g) / p.shape[-1] ** 0.5).to(BF16))
        elif "norm" in name or name.endswith("temp"):
            p.data.fill_(1.0)
        elif name.endswith("A_log"):
            p.data.fill_(-2.0)
    return model


def mopalorn_config(width, heads, vocab=32000):
    """Four layers, one of each kind and a second latent one: windowed attention with pooled blocks and a sink (512 keys + one row per 32 older tokens), latent
    attention (128 + 64 | 128 per head, latent 256, 512-key window, gated), capped attention over all keys with a query temperature, latent attention again;
    grouped queries over 2 key heads; every layer with a dense xIELU feed-forward of ff = 4 width; values mixed from the first layer on."""
    gqa = {"heads": heads, "kv_heads": 2, "dim": 128, "vdim": 128, "scale": 128 ** -0.5, "v_mix": True}
    lat = {"heads": heads, "dim": 128, "rot_dim": 64, "vdim": 128, "kv_rank": 256, "mask": {"size": 512}, "rot": {"dims": 64, "base": 1e6}, "scale": 192 ** -0.5}
    mlp = {"kind": "dense", "ff": 4 * width}
    layers = [{"type": "attention_2", "mixer": dict(gqa, mask={"size": 512, "pool": 32}), "mlp": mlp}, {"type": "latent_attention", "mixer": lat, "mlp": mlp},
              {"type": "attention", "mixer": dict(gqa, q_temp={"coef": 0.25, "every": 128}, softcap=50.0), "mlp": mlp}, {"type": "latent_attention", "mixer": lat, "mlp": mlp}]
    return {"architecture": "Mopalorn", "vocab": vocab, "width": width, "norm": {"eps": 1e-6}, "logit_scale": 0.125, "layers": layers}


def _fill_random(model, device):
    g = torch.Generator(device=device).manual_seed(7)
    for name, p in model.named_parameters():
        if p.dim() >= 2:
            p.data.copy_((torch.randn(p.shape, device=device, generator=g) / p.shape[-1] ** 0.5).to(BF16))
        elif "norm" in name or name.endswith("temp"):
            p.data.fill_(1.0)
        elif name.endswith("lam") or name.endswith("act"):
            p.data.fill_(0.25)
    return model


def random_mopalorn(width, heads, device):
    from llm_quest_amd.mopalorn.mopalorn_model import MopalornConfig, MopalornModel

    with torch.device(device):
        model = MopalornModel(MopalornConfig(mopalorn_config(width, heads)))
    return _fill_random(model, device)


def mepatar_attention_config(width, heads, vocab=32000):
    """The reference beside Mopalorn: four Mepatar layers of sliding-window attention (512 keys + 4 kept, grouped queries over 2 key heads, 128 | 128) with
    the dense gated feed-forward at ff = 8/3 width (as many weights as an un-gated layer of 4 width), no input convolution, norms in one group."""
    att = {"heads": heads, "kv_heads": 2, "dim": 128, "vdim": 128, "mask": {"size": 512, "keep_first": 4}, "rot": {"dims": 64, "base": 1e6}, "scale": 128 ** -0.5}
    layers = [{"type": "attention", "mixer": att, "mlp": {"kind": "dense", "ff": (8 * width // 3 + 63) // 64 * 64}} for _ in range(4)]
    return {"architecture": "Mepatar", "vocab": vocab, "width": width, "norm": {"eps": 1e-6, "groups": 1}, "canon": {"taps": 1}, "embedding": {"scale": 1.0}, "layers": layers}


def bench_mopalorn(width, heads, batch, prompt, steps, warmup, device):
    return bench_ragged(random_mopalorn(width, heads, device), f"mopalorn-w{width}", batch, prompt, steps, warmup)


def bench_mepatar_attention(width, heads, batch, prompt, steps, warmup, device):
    from llm_quest_amd.mepatar.mepatar_model import MepatarConfig, MepatarModel

    with torch.device(device):
        model = MepatarModel(MepatarConfig(mepatar_attention_config(width, heads)))
    return bench_ragged(_fill_random(model, device), f"mepatar-attention-w{width}", batch, prompt, steps, warmup)


def gepilix_config(width, heads, vocab=32000):
    """Four layers: token-shifted decay attention (heads of 64, as many as fill the width), chunked attention (chunks of 512, grouped queries over 2 key heads,
    128 | 128, capped, head gate) beside a recurrent gated unit as wide as the model (16 blocks, 4 taps), windowed attention (512 keys, rotary on 64 entries with
    rescaled frequencies) beside a state-space layer (heads of 64 filling twice the width, state 128, one group, 4 taps), decay attention again; three layers
    with 16 experts (2 per token, ff = 1.75 width) plus a shared expert of the same size, one dense squared-ReLU layer (ff = 3.5 width)."""
    wkv = {"heads": width // 64, "dim": 64}
    att = {"heads": heads, "kv_heads": 2, "dim": 128, "vdim": 128, "mask": {"size": 512}, "scale": 128 ** -0.5, "softcap": 50.0}
    rot = {"dims": 64, "base": 5e5, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}}
    moe = {"kind": "moe", "expert": {"ff": int(width * 1.75)}, "router": {"experts": 16, "top": 2}, "shared": {"ff": int(width * 1.75)}}
    dense = {"kind": "dense", "ff": int(width * 3.5)}
    layers = [{"type": "wkv", "mixer": wkv, "mlp": moe},
              {"type": "parallel", "mixer": {"left": att, "right": {"width": width, "blocks": 16, "conv": 4}}, "mlp": dense},
              {"type": "parallel_2", "mixer": {"left": dict(att, rot=rot), "left_scale": 1.0, "right_scale": 1.0,
                                               "right": {"heads": 2 * width // 64, "vdim": 64, "state": 128, "groups": 1, "norm_groups": 1, "conv": 4}}, "mlp": moe},
              {"type": "wkv", "mixer": wkv, "mlp": moe}]
    return {"architecture": "Gepilix", "vocab": vocab, "width": width, "norm": {"eps": 1e-6}, "layers": layers}


def random_gepilix(width, heads, device, decay_rank=64):
    from llm_quest_amd.gepilix.gepilix_model import GepilixConfig, GepilixModel

    raw = gepilix_config(width, heads)
    with torch.device(device):
        model = GepilixModel(GepilixConfig(raw, {i: decay_rank for i, l in enumerate(raw["layers"]) if l["type"] == "wkv"}))
    g = torch.Generator(device=device).manual_seed(7)
    for name, p in model.named_parameters():
        leaf = name.rsplit(".", 1)[-1]
        if leaf == "conv":
            p.data.copy_((0.3 * torch.randn(p.shape, device=device, generator=g)).to(BF16))
        elif p.dim() >= 2:
            p.data.copy_((torch.randn(p.shape, device=device, generator=g) / p.shape[-1] ** 0.5).to(BF16))
        elif leaf in ("weight", "norm", "ls1", "ls2", "left_out", "right_out", "D"):
            p.data.fill_(1.0)
        elif leaf in ("alpha", "u"):
            p.data.fill_(0.5)
        elif leaf == "w0":
            p.data.fill_(-1.0)
    return model


def bench_gepilix(width, heads, batch, prompt, steps, warmup, device):
    return bench_ragged(random_gepilix(width, heads, device), f"gepilix-w{width}", batch, prompt, steps, warmup)


def _time(fn, warmup, steps):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def bench_gemepel(width, heads, batch, prompt, steps, warmup, device):
    return bench_ragged(random_gemepel(width, heads, device), f"gemepel-w{width}", batch, prompt, steps, warmup)


def bench_mepatar(width, heads, batch, prompt, steps, warmup, device):
    return bench_ragged(random_mepatar(width, heads, device), f"mepatar-w{width}", batch, prompt, steps, warmup)


def bench_ragged(model, name, batch, prompt, steps, warmup):
    from llm_quest_amd.generate import RaggedBatch

    vocab = model.vocab_size
    g = torch.Generator().manual_seed(1)
    prompts = [torch.randint(0, vocab, (prompt,), generator=g).tolist() for _ in range(batch)]
    rb = RaggedBatch(model, max_tokens=prompt + steps + warmup + 8, slots=batch)
    state = {"n": 0}

    def prefill():
        ids = [(state["n"], i) for i in range(batch)]
        state["n"] += 1
        rb.step([(sid, p) for sid, p in zip(ids, prompts)])
        state["last"] = ids

    def close_last():
        for sid in state.pop("last", []):
            rb.finish(sid)

    def prefill_cycle():
        close_last()
        prefill()

    t_prefill = _time(prefill_cycle, max(1, warmup // 2), max(2, steps // 8))
    ids = state["last"]
    tok = [[5]] * batch
    t_decode = _time(lambda: rb.step(list(zip(ids, tok))), warmup, steps)
    close_last()
    # one sequence alone
    rb.step([("solo", prompts[0])])
    t_solo = _time(lambda: rb.step([("solo", [5])]), warmup, steps)
    params = sum(p.numel() for p in model.parameters())
    return {"model": name, "params_M": round(params / 1e6, 1), "prefill_tok_s": round(batch * prompt / t_prefill), "prefill_ms": round(t_prefill * 1e3, 2),
            "decode_tok_s": round(batch / t_decode), "decode_ms_per_step": round(t_decode * 1e3, 3), "decode_b1_ms_per_step": round(t_solo * 1e3, 3)}


def bench_qwen35(width, heads, batch, prompt, steps, warmup, device):
    from llm_quest_amd.config import QWEN3_5_08B_CONFIG
    from llm_quest_amd.qwen.qwen3_5.qwen3_5_text_model import Qwen3_5TextModel
    from llm_quest_amd.utils import Qwen3_5Cache

    cfg = dict(QWEN3_5_08B_CONFIG, vocab_size=32000, emb_dim=width, hidden_dim=int(width * 3.5), n_layers=4, linear_sdpa_ratio=4, n_heads=heads, num_kv_groups=2,
               context_length=prompt + steps + warmup + 64)
    torch.manual_seed(3)
    with torch.device(device):
        model = Qwen3_5TextModel(cfg).eval()
    ids = torch.randint(0, 32000, (batch, prompt), device=device)
    holder = {}

    def prefill():
        holder["c"] = Qwen3_5Cache(cfg["n_layers"], cfg["linear_sdpa_ratio"], prompt, cfg["context_length"])
        with torch.inference_mode():
            model(ids, cache=holder["c"])

    t_prefill = _time(prefill, max(1, warmup // 2), max(2, steps // 8))
    tok = torch.full((batch, 1), 5, device=device)

    def decode():
        with torch.inference_mode():
            model(tok, cache=holder["c"])

    t_decode = _time(decode, warmup, steps)
    ids1 = ids[:1].contiguous()
    holder["c"] = Qwen3_5Cache(cfg["n_layers"], cfg["linear_sdpa_ratio"], prompt, cfg["context_length"])
    with torch.inference_mode():
        model(ids1, cache=holder["c"])
    tok1 = tok[:1].contiguous()

    def decode1():
        with torch.inference_mode():
            model(tok1, cache=holder["c"])

    t_solo = _time(decode1, warmup, steps)
    params = sum(p.numel() for p in model.parameters())
    return {"model": f"qwen3.5-text-w{width}", "params_M": round(params / 1e6, 1), "prefill_tok_s": round(batch * prompt / t_prefill), "prefill_ms": round(t_prefill * 1e3, 2),
            "decode_tok_s": round(batch / t_decode), "decode_ms_per_step": round(t_decode * 1e3, 3), "decode_b1_ms_per_step": round(t_solo * 1e3, 3)}


def run(which, steps, warmup, sizes=((1024, 8), (2048, 16)), batch=8, prompt=1024, device="cuda", with_reference=True):
    benches = {"gemepel": bench_gemepel, "mepatar": bench_mepatar, "mopalorn": bench_mopalorn, "mepatar-attention": bench_mepatar_attention, "gepilix": bench_gepilix}
    if which not in benches:
        raise SystemExit(f"--serve: unknown model {which!r} (known: {sorted(benches)})")
    reference = {"mopalorn": bench_mepatar_attention, "gepilix": bench_mepatar}.get(which, bench_qwen35)
    rows = []
    for width, heads in sizes:
        rows.append(benches[which](width, heads, batch, prompt, steps, warmup, device))
        if with_reference:
            rows.append(reference(width, heads, batch, prompt, steps, warmup, device))
    out = {"metric": "serving throughput (random weights)", "unit": "tokens/s", "batch": batch, "prompt": prompt, "steps": steps, "warmup": warmup,
           "dtype": "bf16", "data": "synthetic", "rows": rows}
    print(json.dumps(out))
    return out

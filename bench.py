"""Decode and prefill throughput of the engine at TinyLlama-1.1B sizes with random weights.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--prompt-len 512] [--layers L]
                  [--sizes tinyllama-1.1b|llama-2-7b|llama-3-8b] [--context-limit 2048] [--prefill-tokens 2048]
                  [--tune-products off|heuristic|all] [--no-points] [--only-prefill]
  python bench.py --design kasuvik|furapel|fisesun|betirax [--design-sizes 2048,4096] [--layers 4] [--prefill-tokens 2048] [--steps K]

A "step" is one decode step of the whole engine (schedule, batch metadata, upload, model step on
the GPU, sampling, download, update).  W untimed steps, then exactly K timed steps between two
device synchronisations.  One JSON line is printed: decoded tokens a second at the default batch,
the same at batch 1 and 64, a 2,048-token prefill, and the decode step's memory roofline.

--design kasuvik leaves that workload alone and measures something else: prefill and decode throughput of the
Kasuvik decoder (attention over a window and pooled blocks beside a selective scan, and delta-rule layers) at
layer sizes that resemble served models, beside the Llama decoder at equal width, heads, feed-forward and
depth, both with random weights through the same engine.  One JSON line with both designs' figures per size.

--design furapel does the same for the Furapel decoder (side-by-side layers with dynamic tanh norms: gated grouped-query
attention, latent attention over a window, a matrix memory with exponential gates, routed experts) beside the Kasuvik
and the Llama decoder at equal width, heads, active feed-forward width and depth.

--design fisesun does the same for the Fisesun decoder (layers that norm a sublayer's output only: grouped-query attention
with q and k normed over the whole projection, capped scores, a window that keeps the first tokens, blended values; a
matrix memory; gated experts named by a table per token id beside a shared expert) beside the Furapel and the Llama decoder.

--design betirax does the same for the Betirax decoder (layers that norm after the sum: grouped-query attention with a norm
per head, keys as values, a query temperature, a distance bias, a window and a gate per element; latent attention with a
rotated key part and query latents; a dense feed-forward or gated experts weighted over the chosen logits beside a shared
expert) beside the Fisesun and the Llama decoder.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# MI355X published peaks
HBM_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp16": 2.5e15, "fp8": 5.0e15, "fp32": 157.3e12}

# TinyLlama-1.1B sizes: 22 layers of width 2048, 32 query heads and 4 key/value heads of 64, SwiGLU width
# 5632, vocabulary 32000, context 2048
SIZES = dict(vocab_size=32000, hidden_size=2048, intermediate_size=5632, num_hidden_layers=22,
             num_attention_heads=32, num_key_value_heads=4, head_dim=64, max_position_embeddings=2048,
             rope_theta=10000.0, rms_norm_eps=1e-5, tie_word_embeddings=False)


def build_engine(cfg, dtype, max_num_seqs, max_batched_tokens, tensors, context_limit=2048, tune_products="off"):
    from kvcm_amd.config.engine_config import EngineConfig
    from kvcm_amd.engine.engine import Engine
    ec = EngineConfig(block_size=16, max_seq_len=context_limit, num_blocks=max_num_seqs * context_limit // 16,
                      max_num_seqs=max_num_seqs, max_batched_tokens=max_batched_tokens, dtype=dtype,
                      max_logit_rows=max(max_num_seqs, 64), tune_products=tune_products,
                      # random weights rotate any position: a context limit beyond the sizes' own is allowed
                      beyond_max_position=context_limit > cfg.max_position_embeddings)
    return Engine(config=ec, architecture="LlamaForCausalLM", model_config=cfg, tensors=tensors)


def prompt_step_count(batch, prompt_len, budget=4096):
    """Steps that the prompts of a batch take at most: whole prompts, as many a step as the token budget
    holds beside the tokens of the requests that decode already."""
    per_step = max(1, (budget - batch) // prompt_len)
    return -(-batch // per_step) + 2


def decode_run(eng, batch, prompt_len, steps, warmup, vocab, seed=1):
    """-> (seconds for `steps` decode steps, mean context length during them)."""
    import numpy as np
    import torch
    rng = np.random.default_rng(seed)
    # requests admitted first decode while the others' prompts still run: room for those steps too
    prompt_steps = prompt_step_count(batch, prompt_len, eng.config.max_batched_tokens)
    for _ in range(batch):
        eng.add_request(rng.integers(3, vocab, size=prompt_len).tolist(), max_new_tokens=warmup + steps + 24 + prompt_steps)
    extra = 0
    while True:                                 # prompts, whole, as many per step as the budget takes
        info = eng.step()
        if info.prefill_tokens == 0 and eng.core.num_waiting() == 0:
            break
        extra += 1
    for _ in range(warmup):
        eng.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        info = eng.step()
        assert info.decode_seqs == batch and info.prefill_tokens == 0, "a timed step was not a pure decode step"
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ctx = prompt_len + 2 + extra / 2.0 + warmup + (steps - 1) / 2.0
    # drain
    while not eng.idle():
        eng.step()
    eng.take_finished()
    return dt, ctx


def prefill_run(eng, tokens, vocab, reps=3):
    import numpy as np
    import torch
    rng = np.random.default_rng(7)
    times = []
    for r in range(reps + 1):
        eng.add_request(rng.integers(3, vocab, size=tokens).tolist(), max_new_tokens=1)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        info = eng.step()
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        assert info.prefill_tokens == tokens
        eng.take_finished()
    return sorted(times[1:])[len(times[1:]) // 2]     # median, first one is warm-up


def measured_peaks():
    """What this GPU does in this run, beside the published peaks: GB/s of a copy kernel (1 GiB read and
    written), GB/s of a read-only kernel over 2 GiB, and TFLOP/s of a loop of bfloat16 matrix instructions
    that touches no memory.  Median of five launches each, timed by device events."""
    import torch
    from kvcm_amd import ops
    src = torch.zeros(1 << 29, dtype=torch.int32, device="cuda:0")       # 2 GiB
    dst = torch.empty(1 << 28, dtype=torch.int32, device="cuda:0")       # 1 GiB
    sink = torch.zeros(256, dtype=torch.float32, device="cuda:0")

    def timed(fn):
        ms = []
        for _ in range(6):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            fn()
            b.record()
            b.synchronize()
            ms.append(a.elapsed_time(b))
        return sorted(ms[1:])[2] * 1e-3

    copy_s = timed(lambda: ops.probe_copy(src[:1 << 28], dst, grid=4096))
    read_s = timed(lambda: ops.probe_read(src, sink, grid=4096))
    flops = []
    mfma_s = timed(lambda: flops.append(ops.probe_mfma(20000, sink, grid=2048)))
    out = {"hbm_copy_GBs": round(2 * (1 << 30) / copy_s / 1e9, 1), "hbm_read_GBs": round((1 << 31) / read_s / 1e9, 1),
           "mfma_bf16_TFLOPs": round(flops[-1] / mfma_s / 1e12, 1)}
    del src, dst
    torch.cuda.empty_cache()
    return out


# ------------------------------------------------------------------ another design beside the Llama decoder
# Layer sizes per width: (heads, kv heads, head size, feed-forward, window, block, scan state, step-size rank, decay rank)
DESIGN_SIZES = {2048: (32, 4, 64, 5632, 512, 64, 16, 128, 64), 4096: (32, 8, 128, 14336, 1024, 64, 16, 256, 64)}


def kasuvik_pair(width, layers, vocab=32000):
    """(Kasuvik configuration, Llama configuration) of equal width, heads, feed-forward, depth and vocabulary; every
    fourth layer of the first is a delta-rule layer (the second of each four), the others are parallel layers."""
    from kvcm_amd.config.kasuvik_config import KasuvikConfig
    from kvcm_amd.config.model_config import LlamaConfig
    nh, nkv, hd, ff, window, pool, state, dt_rank, rank = DESIGN_SIZES[width]
    left = {"heads": nh, "kv_heads": nkv, "dim": hd, "vdim": hd, "conv": 4, "rot": {"dims": hd, "base": 10000.0},
            "scale": hd ** -0.5, "mask": {"size": window, "pool": pool}}
    right = {"inner": 2 * width, "state": state, "dt_rank": dt_rank, "conv": 4}
    listed = []
    for i in range(layers):
        if i % 4 == 1:
            listed.append({"type": "general_delta", "mixer": {"heads": nh, "dim": hd, "rank": rank}, "mlp": {"kind": "dense", "ff": ff}})
        else:
            listed.append({"type": "parallel", "mixer": {"left": left, "right": right}, "mlp": {"kind": "dense", "ff": ff}})
    kas = KasuvikConfig.from_dict({"architecture": "Kasuvik", "vocab": vocab, "width": width, "embedding": {"scale": 1.0},
                                   "norm": {"eps": 1e-6}, "layers": listed})
    llama = LlamaConfig.from_dict(dict(vocab_size=vocab, hidden_size=width, intermediate_size=ff, num_hidden_layers=layers,
                                       num_attention_heads=nh, num_key_value_heads=nkv, head_dim=hd, max_position_embeddings=8192,
                                       rope_theta=10000.0, rms_norm_eps=1e-6, tie_word_embeddings=False))
    return kas, llama


# Furapel at a width: (latent size, window of the latent attention, experts, experts a row); the other sizes are DESIGN_SIZES'
FURAPEL_SIZES = {2048: (128, 512, 8, 2), 4096: (128, 1024, 8, 2)}


def furapel_config(width, layers, vocab=32000):
    """A Furapel configuration at a width of DESIGN_SIZES: layers latent attention, gated attention, matrix memory, gated
    attention in turn, each beside ``experts`` experts of which a row uses ``top`` (together as wide as the dense
    feed-forward of the same width), the first layer led in by the product that mixes the embedding in again."""
    from kvcm_amd.config.furapel_config import FurapelConfig
    nh, nkv, hd, ff = DESIGN_SIZES[width][:4]
    rank, window, experts, top = FURAPEL_SIZES[width]
    mlp = {"kind": "moe", "expert": {"ff": ff // top}, "router": {"experts": experts, "top": top}}
    attention = {"heads": nh, "kv_heads": nkv, "dim": hd, "vdim": hd, "scale": hd ** -0.5,
                 "rot": {"dims": hd // 2, "base": 10000.0, "scaling": {"factor": 4.0, "original": 4096, "fast": 32.0, "slow": 1.0}}}
    latent = {"heads": nh, "dim": hd, "vdim": hd, "kv_rank": rank, "scale": hd ** -0.5, "mask": {"size": window}}
    memory = {"heads": nh, "dim": hd, "vdim": hd, "gate_cap": 15.0}
    kinds = [("latent_attention", latent), ("attention", attention), ("mlstm", memory), ("attention", attention)]
    listed = [{"type": kinds[i % 4][0], "mixer": kinds[i % 4][1], "mlp": mlp} for i in range(layers)]
    return FurapelConfig.from_dict({"architecture": "Furapel", "vocab": vocab, "width": width, "embedding": {"scale": 1.0},
                                    "norm": {"eps": 1e-6}, "logit_scale": 1.0, "layers": listed,
                                    "loop": {"start": 0, "stop": 1, "times": 1}})


# Fisesun at a width: (first tokens a window keeps, cap on the scores, experts, experts a row); the other sizes are DESIGN_SIZES'
FISESUN_SIZES = {2048: (4, 50.0, 8, 2), 4096: (4, 50.0, 8, 2)}


def fisesun_config(width, layers, vocab=32000):
    """A Fisesun configuration at a width of DESIGN_SIZES: layers attention, attention, matrix memory, attention in turn
    (the attention layers blend their values with the first one's), each followed by ``experts`` gated experts of which a
    row uses ``top`` and a shared expert (the ``top`` experts a quarter each and the shared one half of the dense
    feed-forward's width)."""
    from kvcm_amd.config.fisesun_config import FisesunConfig
    nh, nkv, hd, ff, window = DESIGN_SIZES[width][:5]
    keep, cap, experts, top = FISESUN_SIZES[width]
    mlp = {"kind": "moe", "expert": {"ff": ff // (2 * top)}, "router": {"experts": experts, "top": top}, "shared": {"ff": ff // 2}}
    attention = {"heads": nh, "kv_heads": nkv, "dim": hd, "vdim": hd, "scale": hd ** -0.5, "softcap": cap, "v_mix": True,
                 "mask": {"size": window, "keep_first": keep},
                 "rot": {"dims": hd, "base": 500000.0, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}}}
    memory = {"heads": nh, "dim": hd, "vdim": hd, "gate_cap": 15.0}
    kinds = [("attention", attention), ("attention", attention), ("mlstm", memory), ("attention", attention)]
    listed = [{"type": kinds[i % 4][0], "mixer": kinds[i % 4][1], "mlp": mlp} for i in range(layers)]
    return FisesunConfig.from_dict({"architecture": "Fisesun", "vocab": vocab, "width": width, "embedding": {"scale": 1.0},
                                    "norm": {"eps": 1e-6}, "logit_softcap": 30.0, "layers": listed})


# Betirax at a width: (cached latent, rotated key part, query latent, positions per temperature step, experts, experts a row)
BETIRAX_SIZES = {2048: (64, 64, 768, 1024, 8, 2), 4096: (64, 64, 1536, 1024, 8, 2)}


def betirax_config(width, layers, vocab=32000):
    """A Betirax configuration at a width of DESIGN_SIZES: layers attention, attention, latent attention, attention in turn
    (every second latent attention reads the pages of the one before it); the first and third of four are followed by a
    dense feed-forward, the others by ``experts`` gated experts of which a row uses ``top`` and a shared expert (the ``top``
    experts a quarter each and the shared one half of the dense feed-forward's width)."""
    from kvcm_amd.config.betirax_config import BetiraxConfig
    nh, nkv, hd, ff, window = DESIGN_SIZES[width][:5]
    rank, rot, q_rank, every, experts, top = BETIRAX_SIZES[width]
    moe = {"kind": "moe", "expert": {"ff": ff // (2 * top)}, "router": {"experts": experts, "top": top}, "shared": {"ff": ff // 2}}
    dense = {"kind": "dense", "ff": ff}
    attention = {"heads": nh, "kv_heads": nkv, "dim": hd, "vdim": hd, "scale": hd ** -0.5, "mask": {"size": window},
                 "q_temp": {"coef": 0.25, "every": every}}
    latent = {"heads": nh, "dim": hd, "rot_dim": rot, "vdim": hd, "kv_rank": rank, "q_rank": q_rank, "scale": (hd + rot) ** -0.5,
              "rot": {"dims": rot, "base": 10000.0, "scaling": {"factor": 4.0, "original": 4096, "fast": 32.0, "slow": 1.0}}}
    listed, owner = [], None
    for i in range(layers):
        mlp = dense if i % 2 == 0 else moe
        if i % 4 == 2:
            mixer = dict(latent)
            if owner is not None:
                mixer["kv_from"], owner = owner, None
            else:
                owner = i
            listed.append({"type": "latent_attention", "mixer": mixer, "mlp": mlp})
        else:
            listed.append({"type": "attention", "mixer": attention, "mlp": mlp})
    return BetiraxConfig.from_dict({"architecture": "Betirax", "vocab": vocab, "width": width, "embedding": {"scale": 1.0},
                                    "norm": {"eps": 1e-6}, "postln_alpha": 2.0, "layers": listed})


def design_main(args):
    import torch
    from kvcm_amd.config.engine_config import EngineConfig
    from kvcm_amd.engine.engine import Engine
    from kvcm_amd.weights.random_init import random_tensors
    layers = args.layers or 4
    T = args.prefill_tokens
    steps, warmup = min(args.steps, 64), min(args.warmup, 8)
    limit = max(2048, -(-(T + 64) // 64) * 64, -(-(args.prompt_len + steps + warmup + 64) // 64) * 64)
    dt = torch.bfloat16 if args.dtype == "bfloat16" else torch.float32
    key = "bf16" if args.dtype == "bfloat16" else "fp32"
    first = args.design
    record = {"metric": "prefill and decode tok/s of the %s decoder beside the %s at equal sizes"
                        % (first.capitalize(), {"kasuvik": "Llama decoder", "furapel": "Kasuvik and Llama decoders",
                                                 "fisesun": "Furapel and Llama decoders", "betirax": "Fisesun and Llama decoders"}[first]), "dtype": key,
              "data": "synthetic", "layers": layers, "prefill_tokens": T, "prompt_len": args.prompt_len, "steps": steps, "sizes": {}}
    for width in [int(w) for w in args.design_sizes.split(",")]:
        if width not in DESIGN_SIZES:
            print("bench.py: unknown width %d for --design-sizes; known: %s" % (width, sorted(DESIGN_SIZES)))
            sys.exit(2)
        entry = {}
        designs = dict(zip(("kasuvik", "llama"), kasuvik_pair(width, layers)))
        if first == "furapel":
            designs = {"furapel": furapel_config(width, layers), **designs}
        elif first == "fisesun":
            designs = {"fisesun": fisesun_config(width, layers), "furapel": furapel_config(width, layers), "llama": designs["llama"]}
        elif first == "betirax":
            designs = {"betirax": betirax_config(width, layers), "fisesun": fisesun_config(width, layers), "llama": designs["llama"]}
        if args.design_alone:
            designs = {first: designs[first]}
        for name, cfg in designs.items():
            arch = {"kasuvik": "Kasuvik", "furapel": "Furapel", "fisesun": "Fisesun", "betirax": "Betirax", "llama": "LlamaForCausalLM"}[name]
            tensors = random_tensors(arch, cfg, seed=0, dtype=dt, device="cuda:0")
            ec = EngineConfig(block_size=16, max_seq_len=limit, num_blocks=8 * limit // 16, max_num_seqs=8,
                              max_batched_tokens=max(4096, T + 64), dtype=args.dtype, max_logit_rows=64, beyond_max_position=True)
            eng = Engine(config=ec, architecture=arch, model_config=cfg, tensors=tensors)
            del tensors
            V = eng.model.spec.vocab_size
            sec = prefill_run(eng, T, V)
            # (row, key) pairs a prompt's rows see: all earlier tokens, or a window's; Furapel's layers differ (its parts are
            # asked with the full count: its attention layers weigh most)
            flops = eng.model.step_flops(T, 1, T * min(T, DESIGN_SIZES[width][4]) if name == "kasuvik" else T * (T + 1) // 2)
            one = {"prefill_tok_s": round(T / sec, 1), "prefill_ms": round(sec * 1e3, 3),
                   "prefill_flops_frac": round(flops / sec / PEAK_FLOPS[key], 4)}
            for b in (1, 8):
                s, c = decode_run(eng, b, args.prompt_len, steps, warmup, V, seed=20 + b)
                one["decode_b%d_tok_s" % b] = round(b * steps / s, 1)
                one["decode_b%d_ms" % b] = round(1e3 * s / steps, 4)
                one["decode_b%d_hbm_frac" % b] = round(eng.runner.step_bytes([c] * b) / (s / steps) / 1e9 / HBM_GBS, 4)
            entry[name] = one
            del eng
            torch.cuda.empty_cache()
        if args.design_alone:
            record["sizes"][str(width)] = entry
            continue
        entry["prefill_ratio"] = round(entry[first]["prefill_tok_s"] / entry["llama"]["prefill_tok_s"], 3)
        entry["decode_b8_ratio"] = round(entry[first]["decode_b8_tok_s"] / entry["llama"]["decode_b8_tok_s"], 3)
        record["sizes"][str(width)] = entry
    print(json.dumps(record), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=240)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=512)
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the configuration (0 = all)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--sizes", default="tinyllama-1.1b", help="layer sizes by name (tinyllama-1.1b, llama-2-7b, llama-3-8b)")
    ap.add_argument("--tune-products", default="off", choices=["off", "heuristic", "all"],
                    help="which of the vendor library's algorithms the many-row products of prompt steps run: its first "
                         "choice (the engine's default, and this program's: the figures are a default engine's), the "
                         "fastest of its choices, or the fastest of all; timed at a shape's first use, before anything "
                         "is measured (tens of milliseconds per shape: worth it for shapes that run thousands of times)")
    ap.add_argument("--context-limit", type=int, default=0,
                    help="most tokens a request may hold; sizes the cache pool (default: 2,048, or what --prompt-len, "
                         "--warmup and --steps need if that is more)")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 and prefill measurements")
    ap.add_argument("--only-prefill", action="store_true",
                    help="run nothing but the 2,048-token prefill (for a profiler); prints its record alone")
    ap.add_argument("--prefill-tokens", type=int, default=2048,
                    help="tokens of the prefill measurement (2,048 in the record; other lengths for sweeps)")
    ap.add_argument("--design", default="llama", choices=["llama", "kasuvik", "furapel", "fisesun", "betirax"],
                    help="llama: the workload above (the default); kasuvik: prefill and decode of the Kasuvik decoder beside the "
                         "Llama decoder at equal sizes; furapel: the same for the Furapel decoder beside both; "
                         "fisesun: the same for the Fisesun decoder beside the Furapel and the Llama decoder; "
                         "betirax: the same for the Betirax decoder beside the Fisesun and the Llama decoder "
                         "(--design-sizes, --layers, --prefill-tokens, --prompt-len, --steps)")
    ap.add_argument("--design-sizes", default="2048,4096", help="widths of the --design comparison (2048, 4096)")
    ap.add_argument("--design-alone", action="store_true", help="run the --design itself only, not the designs beside it (for a profiler)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this engine runs on one GPU; --gpus N with N > 1 is not supported")
        sys.exit(2)

    if args.design != "llama":
        return design_main(args)

    # a whole prompt fits a step beside the decoding requests
    budget = max(4096, args.prompt_len + args.batch, args.prefill_tokens + 64)
    needed = args.prompt_len + args.warmup + args.steps + 24 + prompt_step_count(args.batch, args.prompt_len, budget)
    limit = args.context_limit or max(2048, -(-needed // 64) * 64, -(-args.prefill_tokens // 64) * 64)
    if needed > limit:
        print("bench.py: --prompt-len %d plus the decoded tokens does not fit --context-limit %d" % (args.prompt_len, limit))
        sys.exit(2)

    import torch
    from kvcm_amd.config.model_config import LlamaConfig
    from kvcm_amd.weights.random_init import random_tensors

    from kvcm_amd.cli.common import NAMED_SIZES
    if args.sizes not in NAMED_SIZES:
        print("bench.py: unknown --sizes %r; known: %s" % (args.sizes, sorted(NAMED_SIZES)))
        sys.exit(2)
    sizes = dict(SIZES if args.sizes == "tinyllama-1.1b" else NAMED_SIZES[args.sizes])
    label = {"tinyllama-1.1b": "TinyLlama-1.1B", "llama-2-7b": "Llama-2-7B", "llama-3-8b": "Llama-3-8B"}.get(args.sizes, args.sizes)
    full_layers = sizes["num_hidden_layers"]
    if args.layers:
        sizes["num_hidden_layers"] = args.layers
    cfg = LlamaConfig.from_dict(sizes)
    dt = torch.bfloat16 if args.dtype == "bfloat16" else torch.float32
    tensors = random_tensors("LlamaForCausalLM", cfg, seed=0, dtype=dt, device="cuda:0")
    key = "bf16" if args.dtype == "bfloat16" else "fp32"
    H, I, V, L = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size, cfg.num_hidden_layers

    def roofline(batch, seconds_per_step, ctx):
        # the bytes are the loaded model's and its cache storages' own count (every weight the step uses once,
        # the embedding rows of its tokens, the keys and values of the live requests), not a formula of sizes
        achieved = eng.runner.step_bytes([ctx] * batch) / seconds_per_step / 1e9
        return {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_GBS, 4)}

    # the pool holds every request of the largest batch at the context limit
    seqs = args.batch if (args.no_points or args.only_prefill) else max(64, args.batch)
    eng = build_engine(cfg, args.dtype, max_num_seqs=seqs, max_batched_tokens=budget, tensors=tensors, context_limit=limit,
                       tune_products=args.tune_products)
    del tensors
    torch.cuda.empty_cache()

    def prefill_record():
        T = args.prefill_tokens
        sec = prefill_run(eng, T, V)
        flops = eng.model.step_flops(T, 1, T * (T + 1) // 2)      # the parts' own count: products, and q.k and p.v
        return {"value": round(T / sec, 1), "tokens": T, "ms": round(sec * 1e3, 3),
                "frac": round(flops / sec / PEAK_FLOPS[key], 4)}

    def tuning_log():   # which shapes were tuned, the first choice's and the kept algorithm's microseconds
        if os.environ.get("KVCM_BENCH_TUNING_LOG"):
            from kvcm_amd import ops
            for row in ops.library_tuning_log:
                print("tuned M=%d N=%d K=%d: %.1f -> %.1f us (%d candidates)" % row, file=sys.stderr)

    if args.only_prefill:
        print(json.dumps({"prefill": prefill_record()}), flush=True)
        tuning_log()
        return

    seconds, ctx = decode_run(eng, args.batch, args.prompt_len, args.steps, args.warmup, V)
    value = args.batch * args.steps / seconds
    out = {
        "metric": "decode tok/s at batch %d (%s sizes, %d-token prompts)" % (args.batch, label, args.prompt_len),
        "value": round(value, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(1e3 * seconds / args.steps, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": key, "data": "synthetic",
        "config": {"model": "%s sizes, random weights N(0,0.02)" % label, "global_batch": args.batch,
                   "seq_len": args.prompt_len, "parallelism": "single GPU", "layers": L, "layers_full": full_layers,
                   "hidden": H, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
                   "head_dim": cfg.head_dim, "intermediate": I, "vocab": V, "kv_block": 16,
                   "context_limit": limit, "generated": args.warmup + args.steps,
                   "tune_products": args.tune_products},
        "roofline": roofline(args.batch, seconds / args.steps, ctx),
    }
    if not args.no_points:
        points = {}
        for b, k in ((1, min(args.steps, 128)), (64, min(args.steps, 64))):
            s, c = decode_run(eng, b, args.prompt_len, k, min(args.warmup, 8), V, seed=10 + b)
            points[f"decode_b{b}"] = round(b * k / s, 1)
            points[f"decode_b{b}_ms"] = round(1e3 * s / k, 4)
            points[f"decode_b{b}_hbm_frac"] = roofline(b, s / k, c)["frac"]
        out["points"] = points
        out["prefill"] = prefill_record()
        # beside the published peaks the fractions above are taken against: what this GPU reached in this run
        out["measured"] = measured_peaks()
    print(json.dumps(out), flush=True)
    tuning_log()


if __name__ == "__main__":
    main()

"""Decode and prefill throughput of the Llama-3.2-1B shape on one MI355X, and the larger
workloads beside it.

    python bench.py --gpus 1 --steps K --warmup W

The headline value is decoded tokens per second at batch 8 with every request near the
benchmark context (4,096 positions): W untimed decode steps, then exactly K timed ones through
the engine (schedule, forward from the paged cache, on-device greedy sampling, token fed
back), bracketed by device synchronisation.  On the same line: a 2,048-token prefill (one
prompt in one step, the best of eight runs, the later of which replay the captured step) with its
fraction of the bf16 matrix peak, the decode step's achieved fraction of the HBM roofline
(bytes that must be read: every weight once plus the live requests' cache), and under
``points`` decode throughput at batch 1, 8, 32 and 64 over 256 new tokens after 512-token prompts,
whatever ``--steps`` says (each with its fraction of the HBM roofline, ``..._frac``, and the mean
context of its timed steps, ``..._ctx``) and, while the time budget lasts (``--extra-seconds``;
``--skip-extra`` leaves them out), three more workloads, each in a fresh model:

* ``serve_3b_...``: 64 requests with prompts of 128 to 2,048 tokens through the engine under
  continuous batching with a token budget of 512 (chunked prefill), 256 new tokens each, at the
  Llama-3.2-3B shape: generated tokens per second from the first arrival to the last end;
* ``long_8b_...``: 32 requests of 8,192 prompt tokens and 128 new tokens each at the
  Llama-3.1-8B shape: the same, plus tokens per second and HBM fraction of the steps that only
  decode (context about 8,256), and the prompt tokens per second of the steps before them;
* ``deep_8b_...``: the whole Llama-3.1-8B shape decoding at batch 4 with 32,768 positions each,
  and one prompt of 8,192 tokens in one step.

Each of them runs as a child process (the commands below): a failure there is reported on
stderr and leaves the headline as it is.
Weights are random (N(0, 0.02)), prompts are uniform random token ids.

    python bench.py --serve --model llama-3.2-3b --max-batched-tokens 512
    python bench.py --serve --model llama-3.1-8b --requests 32 --min-prompt 8192 \\
        --max-prompt 8192 --new-tokens 128 --max-batched-tokens 8192
    python bench.py --model llama-3.1-8b --batch 4 --context 32768 --prefill-tokens 8192 \
        --steps 32 --warmup 4 --skip-points

run one of those workloads alone and print its own JSON line.

    python bench.py --designs [--sizes llama-3.2-1b,llama-3.2-3b] [--layers N]

is another workload again: the Gipotar design (attention beside an RWKV-style time mix, gated
delta rule, clamped gated unit; random weights) at the width, depth, feed-forward width,
vocabulary and attention heads of a Llama preset, beside that preset itself: a prefill of
``--prefill-tokens`` tokens in one step, and decode steps at batch 8 and 64 after 512-token
prompts, each with the bytes a step has to read (weights once, the live requests' cache, and
for Gipotar their state slots read and written) as a fraction of the HBM rate.
``--design bekunex`` (or ``gipotar,bekunex``) times the Bekunex design that way (attention over
a cached latent, selective scan, a routed feed-forward; of the experts' weights a step counts
those that its tokens reach on average, and of a windowed cache the window).
``--design lagedra`` times the Lagedra design (three layers of linear attention with a fixed
decay per head to one of windowed softmax attention behind short convolutions, feed-forwards
that alternate between a routed mixture and a dense GELU unit).
``--design pamolix`` times the Pamolix design (two residual streams mixed by hyper-connections;
layers alternate between attention over every earlier key with biases, head norms and a sink,
every second of them on the keys and values of the one before, and attention with a window of
1,024 that also keeps the first 64 keys, with a gate per head; feed-forwards alternate between a
dense GELU unit and a mixture of squared-ReLU units).  ``--design lagedra,pamolix`` puts it
beside its closest kin."""
import argparse
import copy
import json
import os
import subprocess
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_GBPS = 8000.0            # MI355X HBM3E, published
PEAK_TFLOPS = {"bfloat16": 2500.0, "float32": 157.3}
PAGE = 16


def say(msg: str) -> None:
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


class Shape:
    """Sizes of a preset and the bytes and flops that follow from them."""

    def __init__(self, cfg: dict, elem: int):
        self.cfg = cfg
        self.L, self.H, self.I = cfg["num_hidden_layers"], cfg["hidden_size"], cfg["intermediate_size"]
        self.nh, self.nkv, self.d = (cfg["num_attention_heads"], cfg["num_key_value_heads"],
                                     cfg["head_dim"])
        self.V = cfg["vocab_size"]
        self.layer_params = ((self.nh + 2 * self.nkv) * self.d * self.H + self.H * self.nh * self.d
                             + 3 * self.H * self.I + 2 * self.H)
        # What a decode step reads of the weights: the layers, the final norm and the output
        # head once (tied or not, it is one (V, H) matrix), and one row of the embedding table
        # per request; an untied model's embedding table is otherwise not touched.
        self.step_weight_bytes = (self.L * self.layer_params + self.V * self.H + self.H) * elem
        self.elem = elem
        self.kv_bytes_per_token = 2 * self.L * self.nkv * self.d * elem

    def decode_step_bytes(self, batch: int, mean_context: float) -> float:
        """What a decode step has to read: every weight it uses once and the live requests'
        cache."""
        return (self.step_weight_bytes + batch * self.H * self.elem
                + batch * mean_context * self.kv_bytes_per_token)

    def prefill_flops(self, T: int) -> float:
        linear = 2.0 * T * self.L * (self.layer_params - 2 * self.H)
        attention = 4.0 * self.L * self.nh * self.d * T * (T + 1) / 2
        return linear + attention + 2.0 * self.V * self.H


def build_model(name: str, dtype: str, layers, longest: int):
    import torch
    from rust_llm_inference_server_amd.config import preset_dict
    from rust_llm_inference_server_amd.engine import random_model
    cfg = preset_dict(name)
    full_layers = cfg["num_hidden_layers"]
    if layers:
        cfg["num_hidden_layers"] = layers
    cfg["max_position_embeddings"] = min(cfg["max_position_embeddings"], longest + 64)
    t0 = time.time()
    model = random_model(cfg, seed=0, dtype=dtype, max_positions=cfg["max_position_embeddings"])
    torch.cuda.synchronize()
    say(f"{name} ready in {time.time() - t0:.1f}s")
    return model, cfg, full_layers


def run_requests(model, shape: Shape, reqs, new_tokens: int, budget: int, trials: int = 2) -> dict:
    """``reqs`` through the engine under continuous batching with a token budget of ``budget``
    (chunked prefill), ``new_tokens`` each with seeded temperature sampling; timed from the
    first arrival to the last end (best of ``trials``) on an engine that has captured its
    decode steps before the first arrival, as a server does when it starts (``warm_up_s``).
    Steps that only decode, with every request live, are also timed on their own."""
    import torch
    from rust_llm_inference_server_amd.config import EngineConfig
    from rust_llm_inference_server_amd.engine import Engine
    from rust_llm_inference_server_amd.sampling import SamplingParams
    lens = [len(r) for r in reqs]
    pages = sum(-(-(n + new_tokens) // PAGE) + 1 for n in lens) + 64
    sp = SamplingParams(max_tokens=new_tokens, ignore_eos=True, temperature=0.8, seed=1)
    best = None
    for trial in range(trials):
        engine = Engine(model, EngineConfig(
            max_num_seqs=len(reqs), max_batched_tokens=max(budget, len(reqs)), num_pages=pages,
            block_size=PAGE, max_seq_len=max(lens) + new_tokens + 8))
        torch.cuda.synchronize()
        t_warm = time.perf_counter()
        engine.warm_up()
        torch.cuda.synchronize()
        t_warm = time.perf_counter() - t_warm
        for r in reqs:
            engine.add_request(r, sp)
        decode_s = prefill_s = 0.0
        decode_steps = decode_tokens = 0
        context_sum = 0.0
        torch.cuda.synchronize()
        t0 = last = time.perf_counter()
        while engine.has_work():
            before = copy.copy(engine.stats())
            running = engine.scheduler.num_running
            engine.step()                      # ends with the sampled tokens on the host
            now = time.perf_counter()
            after = engine.stats()
            made = after.generated_tokens - before.generated_tokens
            if after.prefill_tokens != before.prefill_tokens:
                prefill_s += now - last
            elif running == len(reqs) and made == len(reqs):
                decode_s += now - last
                decode_steps += 1
                decode_tokens += made
                context_sum += (sum(lens) + after.generated_tokens) / len(reqs)
            last = now
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        stats = engine.stats()
        generated = stats.generated_tokens
        say(f"  run {trial}: {dt:.3f}s, {stats.steps} steps, {stats.preemptions} preemptions "
            f"(decode steps captured beforehand in {t_warm:.2f}s)")
        result = {
            "seconds": dt, "generated": generated, "prompt_tokens": sum(lens), "steps": stats.steps,
            "preemptions": stats.preemptions, "tok_s": generated / dt, "warm_up_s": t_warm,
            "total_tok_s": (generated + sum(lens)) / dt,
            "prefill_tok_s": stats.prefill_tokens / prefill_s if prefill_s else 0.0,
            "decode_steps": decode_steps,
            "decode_tok_s": decode_tokens / decode_s if decode_s else 0.0,
            "decode_ms": decode_s / decode_steps * 1e3 if decode_steps else 0.0,
        }
        if decode_steps:
            step_bytes = shape.decode_step_bytes(len(reqs), context_sum / decode_steps)
            result["decode_context"] = context_sum / decode_steps
            result["decode_frac"] = step_bytes / (decode_s / decode_steps) / 1e9 / HBM_GBPS
        if best is None or result["seconds"] < best["seconds"]:
            best = result
        del engine
    return best


def gipotar_like(cfg: dict) -> dict:
    """A Gipotar configuration at the sizes of a Llama preset: the same width, depth,
    feed-forward width, vocabulary and attention heads; layers alternate between attention
    beside a time mix (heads of 64) and the gated delta rule (heads of 128), each with a
    feed-forward."""
    W, d = cfg["hidden_size"], cfg["head_dim"]
    mlp = {"kind": "dense", "ff": cfg["intermediate_size"], "limit": 7.0}
    left = {"heads": cfg["num_attention_heads"], "kv_heads": cfg["num_key_value_heads"], "dim": d,
            "vdim": d, "rot": {"dims": d, "base": cfg["rope_theta"]}, "scale": d ** -0.5}
    parallel = {"type": "parallel", "mlp": mlp,
                "mixer": {"left": left, "left_scale": 0.7,
                          "right": {"heads": W // 64, "dim": 64, "rank": 64}, "right_scale": 0.7}}
    heads = max(1, W // 128)
    delta = {"type": "delta", "mlp": mlp,
             "mixer": {"heads": heads, "kv_heads": max(1, heads // 2), "dim": 128, "vdim": 128,
                       "conv": 4}}
    return {"architecture": "Gipotar", "vocab": cfg["vocab_size"], "width": W,
            "embedding": {"scale": 1.0}, "residual_mult": 1.0, "norm": {"eps": 1e-5},
            "logit_softcap": 30.0,
            "layers": [copy.deepcopy(parallel if i % 2 == 0 else delta)
                       for i in range(cfg["num_hidden_layers"])]}


def bekunex_like(cfg: dict) -> dict:
    """A Bekunex configuration at the sizes of a Llama preset: the same width, depth, vocabulary
    and head count; layers cycle through attention over a cached latent with a rotated key part
    (latent of 512, rotated part of 64), a selective scan (2 x width channels, 16 states), the
    windowed kind with sink and gate (window 1,024) and a reader of that layer's latents; every
    layer has 32 experts of an eighth of the preset's feed-forward width, of which a token takes
    six out of two of four groups, and a shared unit of a quarter of it: as many active
    feed-forward weights per token as the preset has."""
    W, d, H = cfg["hidden_size"], cfg["head_dim"], cfg["num_attention_heads"]
    ff = cfg["intermediate_size"]
    mlp = {"kind": "moe", "expert": {"ff": ff // 8},
           "router": {"experts": 32, "groups": {"count": 4, "keep": 2}, "scale": 2.5, "top": 6},
           "shared": {"ff": ff // 4}}
    full = {"type": "latent_attention", "mlp": mlp,
            "mixer": {"heads": H, "dim": d, "rot_dim": 64,
                      "rot": {"dims": 64, "base": cfg["rope_theta"]}, "vdim": d, "kv_rank": 512,
                      "scale": (d + 64) ** -0.5}}
    scan = {"type": "mamba1", "mlp": mlp,
            "mixer": {"inner": 2 * W, "state": 16, "dt_rank": max(1, W // 16), "conv": 4}}

    def windowed(kv_from):
        m = {"heads": H, "dim": d, "vdim": d, "kv_rank": 512, "mask": {"size": 1024},
             "scale": d ** -0.5}
        if kv_from is not None:
            m["kv_from"] = kv_from
        return {"type": "latent_attention_2", "mlp": mlp, "mixer": m}

    layers = []
    for i in range(cfg["num_hidden_layers"]):
        kind = i % 4
        layers.append(copy.deepcopy(full if kind == 0 else scan if kind == 1 else
                                    windowed(None) if kind == 2 else windowed(i - 1)))
    return {"architecture": "Bekunex", "vocab": cfg["vocab_size"], "width": W,
            "norm": {"eps": 1e-5}, "logit_scale": 1.0, "layers": layers}


def lagedra_like(cfg: dict) -> dict:
    """A Lagedra configuration at the sizes of a Llama preset: the same width, depth, vocabulary,
    heads and head size; of every four layers three are linear attention with a fixed decay per
    head and one is windowed softmax attention (window 1,024, four taps, capped scores, rotation
    with stretched frequencies, values mixed with the first such layer's); feed-forwards
    alternate between a mixture of 32 bounded gated units (a quarter of the preset's
    feed-forward width each, four chosen out of two of four groups) and a dense GELU unit of
    one and a half times the preset's width: as many active feed-forward weights per token as
    the preset has."""
    W, d, H = cfg["hidden_size"], cfg["head_dim"], cfg["num_attention_heads"]
    ff = cfg["intermediate_size"]
    moe = {"kind": "moe", "expert": {"ff": ff // 4, "limit": 7.0},
           "router": {"experts": 32, "groups": {"count": 4, "keep": 2}, "top": 4}}
    dense = {"kind": "dense", "ff": ff * 3 // 2}
    lightning = {"heads": H, "dim": d, "vdim": d,
                 "decay": [1.0 - 2.0 ** -(3.0 + 6.0 * h / H) for h in range(H)]}
    attention = {"heads": H, "kv_heads": cfg["num_key_value_heads"], "dim": d, "vdim": d,
                 "conv": 4, "mask": {"size": 1024}, "scale": d ** -0.5, "softcap": 30.0,
                 "v_mix": True,
                 "rot": {"dims": d, "base": cfg["rope_theta"],
                         "scaling": {"factor": 8.0, "original": 4096, "fast": 16.0, "slow": 2.0}}}
    layers = []
    for i in range(cfg["num_hidden_layers"]):
        softmax = i % 4 == 3
        layers.append(copy.deepcopy({"type": "attention" if softmax else "lightning",
                                     "mixer": attention if softmax else lightning,
                                     "mlp": moe if i % 2 == 0 else dense}))
    return {"architecture": "Lagedra", "vocab": cfg["vocab_size"], "width": W,
            "max_positions": cfg["max_position_embeddings"], "norm": {"eps": 1e-6},
            "layers": layers}


def pamolix_like(cfg: dict) -> dict:
    """A Pamolix configuration at the sizes of a Llama preset: the same width, depth, vocabulary,
    heads and head size; two residual streams; even layers see every earlier key (biased
    projections, head norms, the queries' factor, a sink), and every second of them reads the
    keys and values of the one before it; odd layers have a window of 1,024 that keeps the first
    64 keys, whole-head rotation with positions stretched by 4, capped scores and a gate per
    head; feed-forwards alternate between a dense GELU unit of one and a half times the preset's
    width and a mixture of 32 squared-ReLU units (three eighths of the preset's feed-forward
    width each, four chosen): as many active feed-forward weights per token as the preset has."""
    W, d, H = cfg["hidden_size"], cfg["head_dim"], cfg["num_attention_heads"]
    G, ff = cfg["num_key_value_heads"], cfg["intermediate_size"]
    moe = {"kind": "moe", "expert": {"ff": ff * 3 // 8}, "router": {"experts": 32, "top": 4}}
    dense = {"kind": "dense", "ff": ff * 3 // 2}
    first = {"heads": H, "kv_heads": G, "dim": d, "vdim": d, "scale": d ** -0.5,
             "q_temp": {"coef": 0.1, "every": 1024}}
    second = {"heads": H, "kv_heads": G, "dim": d, "vdim": d, "scale": d ** -0.5,
              "mask": {"size": 1024, "keep_first": 64}, "softcap": 30.0,
              "rot": {"dims": d, "base": cfg["rope_theta"], "scaling": {"factor": 4.0}}}
    layers = []
    for i in range(cfg["num_hidden_layers"]):
        if i % 2 == 0:
            mixer = dict(first, kv_from=i - 2) if i % 4 == 2 else dict(first)
            layers.append({"type": "attention", "mixer": mixer, "mlp": copy.deepcopy(dense)})
        else:
            layers.append({"type": "attention_2", "mixer": copy.deepcopy(second),
                           "mlp": copy.deepcopy(moe)})
    return {"architecture": "Pamolix", "vocab": cfg["vocab_size"], "width": W,
            "embedding": {"scale": 1.0}, "norm": {"eps": 1e-6}, "streams": 2, "layers": layers}


def step_bytes_of(model, batch: int, mean_context: float) -> float:
    """What a decode step of any model has to move: every tensor its parts hold once (the
    embedding table only where the head shares it), each live request's cached positions, and
    its state slot read and written."""
    seen, total = set(), 0
    for t in model._tensors():
        if t.data_ptr() not in seen:
            seen.add(t.data_ptr())
            total += t.numel() * t.element_size()
    table = model.embedding.weight
    if model.head.weight.data_ptr() != table.data_ptr():
        total -= table.numel() * table.element_size()
    total -= routed_idle_bytes(model, batch)
    per_position = 0.0                    # every run reads its group's pages, its own or not
    for b in model.bindings:
        if b.group >= 0:
            req = model.cache_groups[b.group].request
            per_position += req.bytes_per_token(model.act_dtype) * (
                min(mean_context, req.window) if req.window else mean_context)
    return total + batch * (per_position + 2 * model.state_bytes)


def routed_idle_bytes(model, batch: int) -> float:
    """The experts' weights that a decode step of ``batch`` tokens does not read: with E experts
    of which every token takes ``top`` at random, E (1 - 1/E)^(batch top) of them stay idle on
    average."""
    idle = 0.0
    for layer in model.layers:
        ff = getattr(layer, "feed_forward", None)
        if ff is not None and hasattr(ff, "experts"):
            E = ff.experts
            up = ff.w_gate_up if hasattr(ff, "w_gate_up") else ff.w_up
            per_expert = (up.numel() + ff.w_down.numel()) * ff.w_down.element_size() / E
            idle += per_expert * E * (1.0 - 1.0 / E) ** (batch * ff.top)
    return idle


def time_prefill(model, prompt, runs: int = 8) -> float:
    """Seconds of one prompt in one step (the best of ``runs``, of which the later ones replay
    the captured step)."""
    import torch
    from rust_llm_inference_server_amd.engine import ModelRunner, StepEntry
    T = len(prompt)
    runner = ModelRunner(model, num_pages=-(-T // PAGE) + 1, page_size=PAGE, max_num_seqs=1)
    times = []
    for _ in range(runs):
        runner.reserve(0, T)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        runner.step([StepEntry(0, prompt, [T - 1])])
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        runner.free(0)
    return min(times[1:] or times)


def time_decode(model, prompts_of_batch, steps: int, warmup: int):
    """(tokens/s, ms/step, mean context) of ``steps`` decode steps of the requests
    ``prompts_of_batch``, all prompts prefilled in one step, the decode steps captured
    beforehand."""
    import torch
    from rust_llm_inference_server_amd.config import EngineConfig
    from rust_llm_inference_server_amd.engine import Engine
    from rust_llm_inference_server_amd.sampling import SamplingParams
    batch, prompt_len = len(prompts_of_batch), len(prompts_of_batch[0])
    new_tokens = steps + warmup + 3
    context = prompt_len + new_tokens
    engine = Engine(model, EngineConfig(
        max_num_seqs=batch, max_batched_tokens=batch * prompt_len,
        num_pages=batch * (-(-context // PAGE) + 1) + 8, block_size=PAGE, max_seq_len=context + 8,
        watermark_pages=0))
    sp = SamplingParams(max_tokens=new_tokens, ignore_eos=True)
    engine.runner.capture_decode_steps(longest=context + 8, max_batch=batch)
    for p in prompts_of_batch:
        engine.add_request(p, sp)
    while engine.stats().prefill_tokens < batch * prompt_len or engine.stats().waiting:
        engine.step()
    for _ in range(warmup):
        engine.step()
    torch.cuda.synchronize()
    before = copy.copy(engine.stats())
    t0 = time.perf_counter()
    for _ in range(steps):
        engine.step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    after = engine.stats()
    if after.generated_tokens - before.generated_tokens != batch * steps:
        raise RuntimeError("the timed steps were not pure decode steps of the whole batch")
    mean_ctx = prompt_len + (before.generated_tokens + after.generated_tokens) / 2 / batch
    return batch * steps / dt, dt / steps * 1e3, mean_ctx


def compare_designs(args) -> int:
    """The Gipotar design beside the Llama preset of the same sizes: one JSON line."""
    import torch
    from rust_llm_inference_server_amd.config import preset_dict
    from rust_llm_inference_server_amd.engine import random_model
    g = torch.Generator().manual_seed(0)
    T, new, warm = args.prefill_tokens, min(args.steps, 64), min(args.warmup, 8)
    results = {}
    for size in args.sizes.split(","):
        base = preset_dict(size)
        if args.layers:
            base["num_hidden_layers"] = args.layers
        longest = max(T, args.points_context + new + warm + 16) + 64
        base["max_position_embeddings"] = min(base["max_position_embeddings"], longest)
        like = {"gipotar": gipotar_like, "bekunex": bekunex_like, "lagedra": lagedra_like,
                "pamolix": pamolix_like}
        for design, cfg in [("llama", base)] + [(d, like[d](base)) for d in args.design.split(",")]:
            vocab = base["vocab_size"]
            model = random_model(cfg, seed=0, dtype=args.dtype, max_positions=longest)
            torch.cuda.synchronize()
            r = {"layers": base["num_hidden_layers"]}
            s = time_prefill(model, torch.randint(0, vocab, (T,), generator=g).tolist())
            r["prefill_tok_s"], r["prefill_ms"] = round(T / s, 1), round(s * 1e3, 3)
            for b in (8, 64):
                reqs = [torch.randint(0, vocab, (args.points_context,), generator=g).tolist()
                        for _ in range(b)]
                v, ms, ctx = time_decode(model, reqs, new, warm)
                frac = step_bytes_of(model, b, ctx) / (ms * 1e-3) / 1e9 / HBM_GBPS
                r[f"decode_b{b}_tok_s"], r[f"decode_b{b}_ms"] = round(v, 1), round(ms, 4)
                r[f"decode_b{b}_hbm_frac"] = round(frac, 4)
            results[f"{size}/{design}"] = r
            say(f"{size} {design}: {r}")
            del model
            torch.cuda.empty_cache()
    print(json.dumps({
        "metric": f"prefill and decode tok/s, {args.design} beside Llama at equal sizes",
        "unit": "tokens/s", "n_gpus": 1, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic (random weights N(0,0.02), uniform random token ids)",
        "config": {"sizes": args.sizes, "prefill_tokens": T, "decode_prompt": args.points_context,
                   "decode_steps": new, "page_size": PAGE},
        "results": results}))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--model", default="llama-3.2-1b", help="preset name")
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the preset")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--points-context", type=int, default=512,
                    help="prompt length of the decode points at batch 1, 8, 32 and 64")
    ap.add_argument("--points-new-tokens", type=int, default=256,
                    help="timed decode steps of each of those points")
    ap.add_argument("--skip-points", action="store_true")
    ap.add_argument("--skip-prefill", action="store_true")
    ap.add_argument("--skip-extra", action="store_true",
                    help="leave out the 3B serving run and the 8B long-context run")
    ap.add_argument("--extra-seconds", type=float, default=150.0,
                    help="an extra workload starts only while the run is younger than this")
    ap.add_argument("--max-batched-tokens", type=int, default=8192,
                    help="token budget of the engine steps that prefill the decode runs")
    ap.add_argument("--serve", action="store_true",
                    help="time a batch of requests through the engine instead")
    ap.add_argument("--requests", type=int, default=64)
    ap.add_argument("--min-prompt", type=int, default=128)
    ap.add_argument("--max-prompt", type=int, default=2048)
    ap.add_argument("--new-tokens", type=int, default=256)
    ap.add_argument("--designs", action="store_true",
                    help="time the Gipotar design beside the Llama presets of --sizes instead")
    ap.add_argument("--design", default="gipotar",
                    help="the designs that --designs times beside Llama, with commas between "
                         "them: gipotar, bekunex, lagedra")
    ap.add_argument("--sizes", default="llama-3.2-1b,llama-3.2-3b",
                    help="presets whose sizes the two designs of --designs are built at")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported (single-GPU engine)")
        return 2
    started = time.time()

    import torch
    from rust_llm_inference_server_amd.config import EngineConfig
    from rust_llm_inference_server_amd.engine import Engine, ModelRunner, StepEntry
    from rust_llm_inference_server_amd.ops import lib
    from rust_llm_inference_server_amd.sampling import SamplingParams

    torch.cuda.set_device(0)
    lib.load()
    K, W = args.steps, args.warmup
    elem = 2 if args.dtype == "bfloat16" else 4
    g = torch.Generator().manual_seed(0)

    def prompts(n, length, vocab):
        return [torch.randint(0, vocab, (length,), generator=g).tolist() for _ in range(n)]

    def random_requests(n, lo, hi, vocab):
        lens = torch.randint(lo, hi + 1, (n,), generator=g).tolist()
        return [torch.randint(0, vocab, (m,), generator=g).tolist() for m in lens]

    if args.designs:
        return compare_designs(args)

    if args.serve:
        # ---- one workload of requests through the engine, alone ------------------------------
        model, cfg, full_layers = build_model(args.model, args.dtype, args.layers,
                                              args.max_prompt + args.new_tokens)
        shape = Shape(cfg, elem)
        reqs = random_requests(args.requests, args.min_prompt, args.max_prompt, shape.V)
        r = run_requests(model, shape, reqs, args.new_tokens, args.max_batched_tokens)
        print(json.dumps({
            "metric": f"served tok/s, {args.requests} requests ({args.model} shape)",
            "value": round(r["tok_s"], 1), "unit": "generated tokens/s", "n_gpus": 1,
            "seconds": round(r["seconds"], 4), "higher_is_better": True,
            "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
            "data": "synthetic (random weights N(0,0.02), uniform random token ids)",
            "config": {"model": args.model, "layers": shape.L, "layers_full": full_layers,
                       "requests": args.requests, "min_prompt": args.min_prompt,
                       "max_prompt": args.max_prompt, "new_tokens": args.new_tokens,
                       "max_batched_tokens": args.max_batched_tokens, "page_size": PAGE,
                       "prompt_tokens": r["prompt_tokens"], "generated_tokens": r["generated"],
                       "steps": r["steps"], "preemptions": r["preemptions"]},
            "total_tokens_per_s": round(r["total_tok_s"], 1),
            "prefill_tokens_per_s": round(r["prefill_tok_s"], 1),
            "warm_up_seconds": round(r["warm_up_s"], 3),
            "decode": {"steps": r["decode_steps"], "tokens_per_s": round(r["decode_tok_s"], 1),
                       "ms_per_step": round(r["decode_ms"], 4),
                       "context": round(r.get("decode_context", 0.0), 1),
                       "hbm_frac": round(r.get("decode_frac", 0.0), 4)},
        }))
        return 0

    # room for the timed steps themselves when they are more than the context holds
    longest = max(args.context, args.prefill_tokens, 4096, K + W + 128)
    model, cfg, full_layers = build_model(args.model, args.dtype, args.layers, longest)
    shape = Shape(cfg, elem)

    def decode_run(batch, context, steps, warmup, prompt_len=None):
        """tokens/s, ms/step and mean context of `steps` decode steps of `batch` requests, none
        of which goes beyond `context` (or, with `prompt_len`, after prompts of that length).
        Prompts are prefilled in portions under the engine's
        token budget while earlier requests already decode, so every request is given room for
        the steps that the prefill of the others takes; the timed steps are pure decode steps."""
        budget = max(args.max_batched_tokens, batch)
        if prompt_len is not None:
            budget = max(budget, batch * prompt_len)      # all prompts in one step
            context = prompt_len
        prefill_steps = -(-batch * context // budget) + 1
        new_tokens = steps + warmup + prefill_steps + 1
        if prompt_len is not None:
            context = prompt_len + new_tokens
        else:
            context = max(context, new_tokens + 16)       # more steps than the context holds
            prompt_len = context - new_tokens
        pages = batch * (-(-context // PAGE) + 1) + 8
        engine = Engine(model, EngineConfig(max_num_seqs=max(batch, 1), max_batched_tokens=budget,
                                            num_pages=pages, block_size=PAGE,
                                            max_seq_len=context + 8, watermark_pages=0))
        sp = SamplingParams(max_tokens=new_tokens, ignore_eos=True)
        # the decode steps' graphs are captured before the first request arrives, as a server
        # does when it starts (Engine.warm_up): the warm-up steps below are then replays
        engine.runner.capture_decode_steps(longest=context + 8, max_batch=batch)
        for p in prompts(batch, prompt_len, shape.V):
            engine.add_request(p, sp)
        while engine.stats().prefill_tokens < batch * prompt_len or engine.stats().waiting:
            engine.step()                                     # prefill, in portions
        for _ in range(warmup):
            engine.step()
        torch.cuda.synchronize()
        before = copy.copy(engine.stats())
        t0 = time.perf_counter()
        for _ in range(steps):
            engine.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        after = copy.copy(engine.stats())
        if (after.generated_tokens - before.generated_tokens != batch * steps
                or after.prefill_tokens != before.prefill_tokens
                or after.preemptions != before.preemptions):
            raise RuntimeError("the timed steps were not pure decode steps of the whole batch")
        mean_ctx = prompt_len + (before.generated_tokens + after.generated_tokens) / 2 / batch
        return batch * steps / dt, dt / steps * 1e3, mean_ctx

    # ---- prefill: one prompt of T tokens in one step, last-row logits ------------------
    T = args.prefill_tokens
    runner = ModelRunner(model, num_pages=-(-T // PAGE) + 1, page_size=PAGE, max_num_seqs=1)
    prompt = prompts(1, T, shape.V)[0]
    times = []
    # (eight: the engine captures a step whose shape has come back three times and replays it
    # from then on, as it does for a server that sees prompts of one length)
    for i in range(1 if args.skip_prefill else 8):
        runner.reserve(0, T)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        runner.step([StepEntry(0, prompt, [T - 1])])
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        runner.free(0)
    prefill_s = min(times[1:] or times)
    prefill = {"value": round(T / prefill_s, 1), "tokens": T, "ms": round(prefill_s * 1e3, 3),
               "frac": round(shape.prefill_flops(T) / prefill_s / (PEAK_TFLOPS[args.dtype] * 1e12), 4)}
    del runner
    say(f"prefill {prefill}")

    # ---- headline: batch B near the benchmark context ------------------------------------
    value, ms_per_step, mean_ctx = decode_run(args.batch, args.context, K, W)
    achieved = shape.decode_step_bytes(args.batch, mean_ctx) / (ms_per_step * 1e-3) / 1e9
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBPS, "unit": "GB/s",
                "frac": round(achieved / HBM_GBPS, 4)}
    say(f"decode b{args.batch}: {value:.0f} tok/s, {ms_per_step:.3f} ms/step, "
        f"{roofline['frac']:.3f} of HBM")

    points = {}
    if not args.skip_points:
        # the metric's own workload: 512-token prompts, then 256 new tokens at batch 1, 8, 32 and 64
        # (after W untimed decode steps, so the timed steps' mean context is 640 + W)
        for b in (1, 8, 32, 64):
            v, ms, mean = decode_run(b, 0, args.points_new_tokens, W, prompt_len=args.points_context)
            frac = shape.decode_step_bytes(b, mean) / (ms * 1e-3) / 1e9 / HBM_GBPS
            name = f"decode_b{b}" if b != args.batch else f"decode_b{b}_p{args.points_context}"
            points[name] = round(v, 1)
            points[name + "_frac"] = round(frac, 4)
            points[name + "_ctx"] = round(mean, 1)
            say(f"decode b{b}, {args.points_new_tokens} new tokens after {args.points_context}-token "
                f"prompts: {v:.0f} tok/s, {ms:.3f} ms/step, {frac:.3f} of HBM at mean context {mean:.0f}")

    # ---- the larger workloads, each in a model of its own ------------------------------------
    extras = [] if args.skip_extra or args.skip_points or args.layers else [
        ("serve_3b", "llama-3.2-3b", dict(n=64, lo=128, hi=2048, new=256, budget=512)),
        ("long_8b", "llama-3.1-8b", dict(n=32, lo=8192, hi=8192, new=128, budget=8192)),
    ]
    if extras:
        extras.append(("deep_8b", "llama-3.1-8b", None))
    for key, name, wl in extras:
        if time.time() - started > args.extra_seconds:
            say(f"{key}: left out, the run is older than {args.extra_seconds:.0f}s")
            continue
        if wl is None:
            # the whole 8B shape: decode at batch 4 with 32,768 positions, a prompt of 8,192
            cmd = [sys.executable, os.path.abspath(__file__), "--model", name, "--dtype", args.dtype,
                   "--batch", "4", "--context", "32768", "--prefill-tokens", "8192", "--steps", "32",
                   "--warmup", "4", "--skip-points"]
            try:
                child = subprocess.run(cmd, stdout=subprocess.PIPE, text=True, timeout=240)
                line = (child.stdout.strip().splitlines() or [""])[-1]
                if child.returncode != 0 or not line.startswith("{"):
                    raise RuntimeError(f"exit code {child.returncode}")
                r = json.loads(line)
                points[f"{key}_b4_ctx32k_tok_s"] = r["value"]
                points[f"{key}_b4_ctx32k_ms"] = r["ms_per_step"]
                points[f"{key}_b4_ctx32k_frac"] = r["roofline"]["frac"]
                points[f"{key}_prefill8192_tok_s"] = r["prefill"]["value"]
                points[f"{key}_prefill8192_frac"] = r["prefill"]["frac"]
                say(f"{key}: batch 4 at 32,768 positions {r['ms_per_step']:.2f} ms/step, "
                    f"{r['roofline']['frac']:.3f} of HBM; prefill of 8,192 tokens "
                    f"{r['prefill']['value']:.0f} tok/s, {r['prefill']['frac']:.3f} of the matrix peak")
            except Exception as exc:
                say(f"{key} failed: {type(exc).__name__}: {exc}")
            continue
        # A process of its own: whatever happens there, the headline below is printed.
        cmd = [sys.executable, os.path.abspath(__file__), "--serve", "--model", name, "--dtype",
               args.dtype, "--requests", str(wl["n"]), "--min-prompt", str(wl["lo"]), "--max-prompt",
               str(wl["hi"]), "--new-tokens", str(wl["new"]), "--max-batched-tokens",
               str(wl["budget"])]
        try:
            child = subprocess.run(cmd, stdout=subprocess.PIPE, text=True, timeout=240)
            line = (child.stdout.strip().splitlines() or [""])[-1]
            if child.returncode != 0 or not line.startswith("{"):
                raise RuntimeError(f"exit code {child.returncode}")
            r = json.loads(line)
            points[f"{key}_tok_s"] = r["value"]
            points[f"{key}_total_tok_s"] = r["total_tokens_per_s"]
            points[f"{key}_prefill_tok_s"] = r["prefill_tokens_per_s"]
            points[f"{key}_decode_tok_s"] = r["decode"]["tokens_per_s"]
            points[f"{key}_decode_ms"] = r["decode"]["ms_per_step"]
            points[f"{key}_decode_frac"] = r["decode"]["hbm_frac"]
            say(f"{key}: {r['value']:.0f} generated tok/s in {r['seconds']:.2f}s; decode steps "
                f"{r['decode']['ms_per_step']:.2f} ms, {r['decode']['tokens_per_s']:.0f} tok/s, "
                f"{r['decode']['hbm_frac']:.3f} of HBM at context {r['decode']['context']:.0f}; "
                f"prompts {r['prefill_tokens_per_s']:.0f} tok/s")
        except Exception as exc:
            say(f"{key} failed: {type(exc).__name__}: {exc}")

    print(json.dumps({
        "metric": f"decode tok/s at batch {args.batch} ({args.model} shape)", "value": round(value, 1),
        "unit": "tokens/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic (random weights N(0,0.02), uniform random token ids)",
        "config": {"model": args.model, "layers": shape.L, "layers_full": full_layers,
                   "hidden": shape.H, "heads": shape.nh, "kv_heads": shape.nkv, "head_dim": shape.d,
                   "intermediate": shape.I, "vocab": shape.V, "global_batch": args.batch,
                   "seq_len": args.context, "page_size": PAGE, "prefill_tokens": T,
                   "points_prompt": args.points_context, "points_new_tokens": args.points_new_tokens,
                   "parallelism": "single GPU"},
        "prefill": prefill, "roofline": roofline, "points": points,
    }))
    return 0


if __name__ == "__main__":
    sys.exit(main())

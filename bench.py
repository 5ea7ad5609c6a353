#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X.

Default: the Qwen3-8B shape (36 layers, hidden 4096, 32 query and
8 key/value heads of 128, intermediate 12288, vocabulary 151936, untied head) with random
bfloat16 weights; 8 requests with 1024-token random prompts decode through the engine's own step
(scheduler, step function, cache, kernels, device sampling).  A "step" is one decode step.
The timed steps are centred on the workload's mean context: with 1024-token prompts and 256 generated tokens
(``--gen-len``) that is 1152 tokens, so untimed steps run up to context 1152 - steps / 2 first, whatever ``--steps`` is.
Prints ONE JSON line: decoded tokens per second, plus the prefill of 2048 tokens, the decode
step's HBM roofline, and decode at batch 1, 32 and 64 and at batch 32 with prompts of uneven lengths (128 to 2048
tokens, ``--uneven``) (tokens per second under "points"; their time per step,
mean context and share of the HBM roofline under "points_detail").  Beside the fractions of the published peaks
(8 TB/s, 2.5 PFLOP/s) the line gives fractions of rates measured at start-up on this GPU: a plain read of 2 GB
("measured_read_gbs", "frac_of_measured") and the library's product of 2048 rows with the model's gate/up matrix
("library_tflops", "frac_of_library").

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B] [--dtype bfloat16|float32]

Other workloads, each again one JSON line:

    python bench.py --shape 14b --serve 64                 # Qwen3-14B shape: 64 requests at once until all have ended
    python bench.py --shape 32b --batch 64 --prompt-len 4096 --context 4608 --points "" --steps 32 --warmup 4   # long keys at the 32B shape
    python bench.py --design sefevik [--design-sizes 1024,2048,4096] [--layers 8]   # Sefevik beside Qwen3 at equal size
    python bench.py --design sodedra [--design-sizes 1024,2048,4096] [--layers 8]   # Sodedra beside Qwen3 at equal size
    python bench.py --design meronex [--design-sizes 1024,2048,4096] [--layers 9]   # Meronex beside Sodedra and Qwen3 at equal size
    python bench.py --design tarunex [--design-sizes 1024,2048,4096] [--layers 8]   # Tarunex beside Sodedra, Sefevik and Qwen3 at equal size
"""
import argparse
import json
import sys
import time

PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bfloat16": 2.5e15, "float32": 157.3e12}

MODEL_8B = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", hidden_act="silu", num_hidden_layers=36, hidden_size=4096,
                num_attention_heads=32, num_key_value_heads=8, head_dim=128, intermediate_size=12288, vocab_size=151936,
                rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=40960,
                bos_token_id=151643, eos_token_id=151645)
# the larger shapes; the default stays the 8B shape
SHAPES = {
    # the size of model that the reference's own run script names (run.sh:2): 28 narrow layers, where a step is many short kernels
    "0.6b": ("Qwen3-0.6B shape", dict(MODEL_8B, num_hidden_layers=28, hidden_size=1024, num_attention_heads=16, intermediate_size=3072,
                                      tie_word_embeddings=True)),
    "1.7b": ("Qwen3-1.7B shape", dict(MODEL_8B, num_hidden_layers=28, hidden_size=2048, num_attention_heads=16, intermediate_size=6144,
                                      tie_word_embeddings=True)),
    "4b": ("Qwen3-4B shape", dict(MODEL_8B, num_hidden_layers=36, hidden_size=2560, num_attention_heads=32, intermediate_size=9728,
                                  tie_word_embeddings=True)),
    "8b": ("Qwen3-8B shape", MODEL_8B),
    "14b": ("Qwen3-14B shape", dict(MODEL_8B, num_hidden_layers=40, hidden_size=5120, num_attention_heads=40, intermediate_size=17408)),
    "32b": ("Qwen3-32B shape", dict(MODEL_8B, num_hidden_layers=64, hidden_size=5120, num_attention_heads=64, intermediate_size=25600)),
}


def sefevik_shape(width: int, layers: int, vocab: int, window: int = 1024) -> dict:
    """A Sefevik configuration with the layer sizes of a real model of that width: heads of 128 unrotated and 64 rotated
    dims, a latent of 512, a feed-forward of three times the width; of every four layers one latent attention with its
    own rows, two recurrences and one latent attention that reads the first one's rows."""
    heads = max(1, width // 128)
    rot = dict(base=10000.0, dims=64, scaling=dict(factor=8.0, original=4096, fast=16.0, slow=2.0))
    att = dict(heads=heads, dim=128, rot_dim=64, vdim=128, kv_rank=512, scale=192 ** -0.5, mask=dict(size=window), rot=rot)
    out = []
    for i in range(layers):
        kind = i % 4
        if kind == 0:
            out.append(dict(type="latent_attention", mixer=dict(att), mlp=dict(kind="dense", ff=3 * width)))
        elif kind == 3:
            out.append(dict(type="latent_attention", mixer=dict(att, kv_from=i - 3), mlp=dict(kind="dense", ff=3 * width)))
        else:
            out.append(dict(type="mingru", mixer=dict(width=width), mlp=dict(kind="dense", ff=3 * width)))
    return dict(architecture="Sefevik", vocab=vocab, width=width, norm=dict(eps=1e-6),
                embedding=dict(bigram=dict(buckets=65521, mul_prev=37, mul_cur=11)), layers=out)


def sodedra_shape(width: int, layers: int, vocab: int, window: int = 1024) -> dict:
    """A Sodedra configuration with the layer sizes of a real model of that width: attention heads of 128 with 64 rotated
    dims and a quarter as many kv heads; matrix memories with keys of 128 (mLSTM: values of 256, half as many heads); a
    dense feed-forward of three times the width, or 32 experts of a quarter of that of which a token uses four (as many
    active weights); of every four layers an mLSTM, an attention with experts, a delta rule and an attention."""
    heads = max(1, width // 128)
    rot = dict(base=500000.0, dims=64, scaling=dict(factor=8.0, low=1.0, high=4.0, original=8192))
    att = dict(heads=heads, kv_heads=max(1, heads // 4), dim=128, vdim=128, scale=128 ** -0.5, mask=dict(size=window), rot=rot)
    dense = dict(kind="dense", ff=3 * width)
    moe = dict(kind="moe", expert=dict(ff=3 * width // 4), router=dict(experts=32, top=4, scale=1.5, groups=dict(count=4, keep=2)))
    out = []
    for i in range(layers):
        kind = i % 4
        if kind == 0:
            out.append(dict(type="mlstm", mixer=dict(heads=max(1, heads // 2), dim=128, vdim=256, gate_cap=16.0), mlp=dense))
        elif kind == 1:
            out.append(dict(type="attention", mixer=dict(att), mlp=moe))
        elif kind == 2:
            out.append(dict(type="channel_delta", mixer=dict(heads=heads, kv_heads=max(1, heads // 2), dim=128, vdim=128, conv=4,
                                                             decay_rank=128, gate_rank=128), mlp=dense))
        else:
            out.append(dict(type="attention", mixer=dict(att), mlp=dense))
    return dict(architecture="Sodedra", vocab=vocab, width=width, norm=dict(eps=1e-6), embedding=dict(scale=1.0), layers=out)


def meronex_shape(width: int, layers: int, vocab: int) -> dict:
    """A Meronex configuration with the layer sizes of a real model of that width: of every three layers an mLSTM (keys
    of 128, values of 256, half as many heads), a delta rule with one decay per head (heads of 128 x 128, half as many q/k
    heads, 4 taps) and an attention (heads of 128 with 64 rotated dims, a quarter as many kv heads, capped scores) beside
    a time mix (heads of 64, a decay of inner size 64); every feed-forward 32 experts of 3/4 width of which a token uses
    four (as many active weights as a dense layer of three times the width); norms in 8 groups."""
    heads = max(1, width // 128)
    rot = dict(base=500000.0, dims=64, scaling=dict(factor=8.0, original=8192, fast=32.0, slow=1.0))
    left = dict(heads=heads, kv_heads=max(1, heads // 4), dim=128, vdim=128, scale=128 ** -0.5, softcap=30.0, rot=rot)
    moe = dict(kind="moe", expert=dict(ff=3 * width // 4, limit=7.0), router=dict(experts=32, top=4))
    out = []
    for i in range(layers):
        kind = i % 3
        if kind == 0:
            out.append(dict(type="mlstm", mixer=dict(heads=max(1, heads // 2), dim=128, vdim=256, gate_cap=16.0), mlp=moe))
        elif kind == 1:
            out.append(dict(type="delta", mixer=dict(heads=heads, kv_heads=max(1, heads // 2), dim=128, vdim=128, conv=4), mlp=moe))
        else:
            out.append(dict(type="parallel", mixer=dict(left=dict(left), right=dict(heads=max(1, width // 64), dim=64, decay_rank=64)), mlp=moe))
    return dict(architecture="Meronex", vocab=vocab, width=width, norm=dict(eps=1e-5, groups=8), residual_mult=0.7, layers=out)


def tarunex_shape(width: int, layers: int, vocab: int) -> dict:
    """A Tarunex configuration with the layer sizes of a real model of that width and ``layers`` layer RUNS: two layers
    fewer are stored, and the first two are walked twice.  Of every three stored layers an attention (heads of 128, a
    quarter as many kv heads, capped scores, temperature steps of 256 positions), a latent attention (heads of 128
    unrotated and 64 rotated dims, a latent of 512, queries through a vector of 3/8 of the width) and an attention;
    every feed-forward 32 experts of half the width of which a token uses four, plus an expert of the width for everyone
    (as many active weights as a dense layer of three times the width)."""
    heads = max(1, width // 128)
    att = dict(heads=heads, kv_heads=max(1, heads // 4), dim=128, vdim=128, scale=128 ** -0.5, softcap=50.0, q_temp=dict(coef=0.2, every=256))
    lat = dict(heads=heads, dim=128, rot_dim=64, vdim=128, kv_rank=512, q_rank=max(128, 3 * width // 8), scale=192 ** -0.5,
               rot=dict(base=10000.0, dims=64))
    moe = dict(kind="moe", expert=dict(ff=width // 2), router=dict(experts=32, top=4), shared=dict(ff=width))
    stored = max(2, layers - 2)
    out = [dict(type="latent_attention", mixer=dict(lat), mlp=moe) if i % 3 == 1 else dict(type="attention", mixer=dict(att), mlp=moe)
           for i in range(stored)]
    return dict(architecture="Tarunex", vocab=vocab, width=width, norm=dict(eps=1e-6), embedding=dict(scale=8.0), logit_scale=0.25,
                logit_softcap=50.0, loop=dict(start=0, stop=2, times=2), layers=out)


DESIGN_SHAPES = {"sefevik": ("Sefevik", sefevik_shape), "sodedra": ("Sodedra", sodedra_shape), "meronex": ("Meronex", meronex_shape),
                 "tarunex": ("Tarunex", tarunex_shape)}
#: further designs that a design is measured beside (Qwen3 always is): the closest ones the engine has
DESIGN_BESIDE = {"meronex": ("sodedra",), "tarunex": ("sodedra", "sefevik")}
#: layers, where --layers does not say: a whole number of the design's turns of layer kinds
DESIGN_LAYERS = {"meronex": 9}


def design_compare(args) -> int:
    """Prefill (one portion of --prefill-tokens) and decode (batch 8 and 32, prompts of --prompt-len) of the design and of
    Qwen3 at equal width, layers, heads and feed-forward size; ONE JSON line."""
    design, (design_name, shape_of) = args.design, DESIGN_SHAPES[args.design]
    import torch

    from spyinfer_amd.config.registry import architecture_of
    from spyinfer_amd.engine.batch import StepEntry
    from spyinfer_amd.engine.llm_engine import LLMEngine
    from spyinfer_amd.engine.runner import bind_weights
    from spyinfer_amd.kernels import ops
    from spyinfer_amd.sampling import SamplingParams
    from spyinfer_amd.weights.random_init import random_tensors_on_device

    ops.hip()
    dev = torch.device("cuda:0")
    layers, vocab, page = args.layers or DESIGN_LAYERS.get(design, 8), 32768, 16
    run_dtype = torch.bfloat16 if args.dtype == "bfloat16" else torch.float32
    g = torch.Generator().manual_seed(args.seed)
    results = {}
    for width in [int(x) for x in args.design_sizes.split(",") if x.strip()]:
        heads = max(1, width // 128)
        raws = {design: shape_of(width, layers, vocab)}
        raws.update({other: DESIGN_SHAPES[other][1](width, layers, vocab) for other in DESIGN_BESIDE.get(design, ())})
        raws.update({"qwen3": dict(MODEL_8B, num_hidden_layers=layers, hidden_size=width, num_attention_heads=heads,
                              num_key_value_heads=max(1, heads // 4), intermediate_size=3 * width, vocab_size=vocab)})
        for name, raw in raws.items():
            arch = architecture_of(raw)
            cfg = arch.config_cls.from_dict(raw)
            model = arch.build(cfg)
            weights = random_tensors_on_device(model.weight_specs(), args.seed, run_dtype, dev)
            params = sum(w.numel() for w in weights.values())
            bind_weights(model, weights, dev, "both")
            del weights
            eng = LLMEngine.__new__(LLMEngine)
            eng._init_with_model(model, dev, dtype=args.dtype, max_model_len=args.context, kvcache_block_size=page,
                                 num_kvcache_blocks=-(-args.context // page) * 32 + 8, max_num_seqs=32,
                                 max_num_batched_tokens=max(16384, args.prefill_tokens), enforce_eager=args.enforce_eager, seed=args.seed)
            out = {"parameters": params}
            T = args.prefill_tokens
            best = None
            for _ in range(4):
                rc = eng.runner.manager.admit("prefill")
                eng.runner.manager.reserve(rc, T)
                toks = torch.randint(0, vocab, (T,), generator=g).tolist()
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                eng.runner.step([StepEntry(rc, toks, [T - 1])])
                torch.cuda.synchronize()
                dt = time.perf_counter() - t0
                eng.runner.manager.release(rc)
                best = dt if best is None else min(best, dt)
            out["prefill_%d" % T] = {"tokens_per_s": round(T / best, 1), "ms": round(best * 1e3, 3)}
            for batch in (8, 32):
                steps, warm = max(16, args.steps // 4), 8
                ids = [eng.add_request(torch.randint(0, vocab, (args.prompt_len,), generator=g).tolist(),
                                       SamplingParams(temperature=0.0, max_new_tokens=steps + warm + 32, ignore_eos=True)) for _ in range(batch)]
                while any(s.is_prefill or s.num_generated == 0 for s in (eng._sequences[i] for i in ids)):
                    eng.step()
                for _ in range(warm):
                    eng.step()
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(steps):
                    assert len(eng.step()) == batch
                torch.cuda.synchronize()
                dt = time.perf_counter() - t0
                for i in ids:
                    eng.remove_request(i)
                out["decode_b%d" % batch] = {"tokens_per_s": round(batch * steps / dt, 1), "ms_per_step": round(dt / steps * 1e3, 4)}
            results.setdefault(str(width), {})[name] = out
            del eng, model
            torch.cuda.empty_cache()
    first = results[next(iter(results))]
    print(json.dumps({
        "metric": "prefill and decode tok/s of %s beside Qwen3 at equal width, layers, heads and feed-forward size" % design_name,
        "value": first[design]["decode_b8"]["tokens_per_s"], "unit": "tokens/s", "n_gpus": 1, "steps": max(16, args.steps // 4), "warmup": 8,
        "ms_per_step": first[design]["decode_b8"]["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic (random weights, uniform-random token ids)",
        "config": {"model": "%s / Qwen3 layer shapes" % design_name, "layers": layers, "vocab": vocab, "prompt_len": args.prompt_len,
                   "prefill_tokens": args.prefill_tokens, "window": 1024, "graphs": not args.enforce_eager, "parallelism": "single GPU"},
        "widths": results}))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (both numbers are reported)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=1024)
    ap.add_argument("--gen-len", type=int, default=256,
                    help="tokens that the workload generates per request: the timed steps are centred on its mean context")
    ap.add_argument("--context", type=int, default=4096, help="max_model_len")
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--points", default="1,32,64", help="further decode batch sizes to report (empty: none)")
    ap.add_argument("--uneven", default="32", help="decode batch sizes to report with prompts of uneven lengths, uniform in "
                                                   "128 .. 2 x prompt-len (empty: none)")
    ap.add_argument("--spread", action="store_true", help="the headline batch's prompts too have uneven lengths (128 .. 2 x prompt-len)")
    ap.add_argument("--even-key-parts", action="store_true",
                    help="every request's keys in one number of parts instead of the host's cut by the step's lengths (for comparison)")
    ap.add_argument("--enforce-eager", action="store_true")
    ap.add_argument("--weight-copies", default="both", choices=["both", "tiled"], help="EngineConfig.weight_copies")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--shape", default="8b", choices=sorted(SHAPES), help="layer sizes of the model")
    ap.add_argument("--serve", type=int, default=0, metavar="N",
                    help="instead of the decode steps: N requests arriving at once, prompts of 128..2048 and outputs of 64..512 "
                         "tokens (uniform), run until all have ended; the value is generated tokens per second of the whole run")
    ap.add_argument("--design", default="", choices=["", "sefevik", "sodedra", "meronex", "tarunex"],
                    help="instead of the decode steps: prefill and decode throughput of that design at a few layer sizes "
                         "beside the Qwen3 shape of equal width, layers, heads and feed-forward size (--design-sizes)")
    ap.add_argument("--design-sizes", default="1024,2048,4096", help="widths for --design")
    args = ap.parse_args()
    if args.design:
        return design_compare(args)
    if args.gpus != 1:
        print("bench.py: this engine runs on one GPU; --gpus %d is not supported" % args.gpus)
        return 2

    import torch

    from spyinfer_amd.config.registry import architecture_of
    from spyinfer_amd.engine.batch import StepEntry
    from spyinfer_amd.engine.llm_engine import LLMEngine
    from spyinfer_amd.engine.runner import bind_weights
    from spyinfer_amd.kernels import ops
    from spyinfer_amd.sampling import SamplingParams
    from spyinfer_amd.weights.random_init import random_tensors_on_device

    ops.hip()
    if args.even_key_parts:
        ops.DECODE_PIECES = False
    dev = torch.device("cuda:0")
    shape_name, shape = SHAPES[args.shape]
    raw = dict(shape)
    model_layers = raw["num_hidden_layers"]
    if args.layers:
        raw["num_hidden_layers"] = args.layers
    arch = architecture_of(raw)
    cfg = arch.config_cls.from_dict(raw)
    model = arch.build(cfg)
    run_dtype = torch.bfloat16 if args.dtype == "bfloat16" else torch.float32
    weights = random_tensors_on_device(model.weight_specs(), args.seed, run_dtype, dev)
    bind_weights(model, weights, dev, args.weight_copies)
    del weights
    torch.cuda.empty_cache()

    points = [int(x) for x in args.points.split(",") if x.strip()]
    uneven = [int(x) for x in args.uneven.split(",") if x.strip()]
    max_batch = max([args.batch, args.serve] + points + uneven)
    page = 16
    pages_per_req = -(-args.context // page)
    eng = LLMEngine.__new__(LLMEngine)
    eng._init_with_model(model, dev, dtype=args.dtype, max_model_len=args.context, kvcache_block_size=page,
                         num_kvcache_blocks=max(pages_per_req * max_batch, -(-args.prefill_tokens // page)) + 8, max_num_seqs=max_batch,
                         max_num_batched_tokens=max(16384, args.prefill_tokens), enforce_eager=args.enforce_eager, seed=args.seed,
                         weight_copies=args.weight_copies)
    g = torch.Generator().manual_seed(args.seed)

    def prompts(n, length):
        return [torch.randint(0, cfg.vocab_size, (length,), generator=g).tolist() for _ in range(n)]

    act_bytes = 2 if args.dtype == "bfloat16" else 4
    L, H, I, V = cfg.num_hidden_layers, cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    nq, nkv, d = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    layer_params = H * (nq + 2 * nkv) * d + nq * d * H + 3 * H * I + 2 * H + 2 * d
    weight_bytes = (L * layer_params + H + V * H) * act_bytes              # every weight a decode step uses, once
    kv_bytes_per_token = sum(s.page_bytes(1, run_dtype) for s in model.cache_specs() if s is not None and s.paged)

    def decode_run(batch, steps, warmup, lengths=None):
        """tokens/s, ms/step, mean context over the timed steps.  Untimed steps first, ``warmup`` at least, until the
        timed window is centred on the workload's mean context (prompt + gen_len / 2).  ``lengths``: the prompts'
        lengths, if not all ``--prompt-len``."""
        lengths = [args.prompt_len] * batch if lengths is None else lengths
        untimed = max(warmup, min((args.gen_len - steps) // 2, args.context - max(lengths) - steps - 2))
        ids = [eng.add_request(prompts(1, n)[0], SamplingParams(temperature=0.0, max_new_tokens=untimed + steps + 64, ignore_eos=True))
               for n in lengths]
        while any(s.is_prefill or s.num_generated == 0 for s in (eng._sequences[i] for i in ids)):
            eng.step()                                                       # prompts, in portions under the budget
        for _ in range(untimed):
            eng.step()
        ctx0 = sum(len(eng._sequences[i]) for i in ids) / batch
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            out = eng.step()
            assert len(out) == batch
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        ctx1 = sum(len(eng._sequences[i]) for i in ids) / batch
        for i in ids:
            eng.remove_request(i)
        return batch * steps / dt, dt / steps * 1e3, (ctx0 + ctx1) / 2

    def prefill_run(tokens, repeats=3):
        best = None
        for _ in range(repeats + 1):
            rc = eng.runner.manager.admit("prefill")
            eng.runner.manager.reserve(rc, tokens)
            toks = prompts(1, tokens)[0]
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            logits = eng.runner.step([StepEntry(rc, toks, [tokens - 1])])
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            eng.runner.manager.release(rc)
            assert logits.shape == (1, V)
            best = dt if best is None else min(best, dt)       # the first run also warms the library up
        return best

    def serve_run(n):
        """n requests at once through the scheduler until all have ended: (generated tokens/s, seconds, steps, mean number
        of requests in a step, preemptions, prompt tokens, generated tokens)."""
        lens = torch.randint(128, 2049, (n,), generator=g).tolist()
        outs = torch.randint(64, 513, (n,), generator=g).tolist()
        for length, new in zip(lens, outs):
            eng.add_request(prompts(1, length)[0], SamplingParams(temperature=0.0, max_new_tokens=new, ignore_eos=True))
        steps = rows = 0
        before = eng.scheduler.num_preemptions
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        while eng.has_unfinished_requests():
            rows += len(eng.step())
            steps += 1
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        return sum(outs) / dt, dt, steps, rows / max(1, steps), eng.scheduler.num_preemptions - before, sum(lens), sum(outs)

    if args.serve:
        serve_run(min(args.serve, 4))                                        # warms the library and the graphs up
        v, dt, steps, mean_rows, pre, n_prompt, n_out = serve_run(args.serve)
        print(json.dumps({
            "metric": "generated tok/s, %d requests at once (%s, prompts 128..2048, outputs 64..512)" % (args.serve, shape_name),
            "value": round(v, 1), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": 0, "ms_per_step": round(dt / steps * 1e3, 4),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
            "data": "synthetic (random weights, uniform-random token ids and lengths)",
            "config": {"model": shape_name, "layers": cfg.num_hidden_layers, "layers_of_model": model_layers, "hidden": cfg.hidden_size,
                       "q_heads": nq, "kv_heads": nkv, "head_dim": d, "intermediate": I, "vocab": V, "global_batch": args.serve,
                       "seq_len": args.context, "prompt_tokens": n_prompt, "generated_tokens": n_out, "seconds": round(dt, 3),
                       "mean_rows_per_step": round(mean_rows, 2), "preemptions": pre, "page_size": page, "parallelism": "single GPU"}}))
        return 0

    # what this GPU gives a kernel that only reads, and the library a product of the prefill's shape: the rates that the
    # decode step and the prefill are held against beside the published peaks
    read_gbs = ops.measure_read_rate(dev) / 1e9
    lib_flops = None
    if args.dtype == "bfloat16":
        a = torch.randn((args.prefill_tokens, H), dtype=torch.bfloat16, device=dev)
        b = torch.randn((2 * I, H), dtype=torch.bfloat16, device=dev)
        best = None
        for _ in range(6):
            t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            t0.record()
            torch.matmul(a, b.t())
            t1.record()
            t1.synchronize()
            best = t0.elapsed_time(t1) if best is None else min(best, t0.elapsed_time(t1))
        lib_flops = 2.0 * args.prefill_tokens * 2 * I * H / (best * 1e-3)
        del a, b
    spread = lambda b: torch.randint(128, min(2 * args.prompt_len, args.context - args.gen_len) + 1, (b,), generator=g).tolist()
    value, ms, ctx = decode_run(args.batch, args.steps, args.warmup, spread(args.batch) if args.spread else None)
    step_bytes = weight_bytes + args.batch * ctx * kv_bytes_per_token
    achieved = step_bytes / (ms * 1e-3) / 1e9
    pf = prefill_run(args.prefill_tokens)
    T = args.prefill_tokens
    linear_flops = 2 * T * L * (H * (nq + 2 * nkv) * d + nq * d * H + 3 * H * I) + 2 * V * H
    attn_flops = L * 4 * d * nq * T * (T + 1) / 2
    pf_flops = linear_flops + attn_flops
    extra, detail = {}, {}
    for b in points:
        v, b_ms, b_ctx = decode_run(b, max(20, args.steps // 2), max(4, args.warmup // 2))
        extra["decode_b%d" % b] = round(v, 1)
        b_gbs = (weight_bytes + b * b_ctx * kv_bytes_per_token) / (b_ms * 1e-3) / 1e9
        detail["decode_b%d" % b] = {"ms_per_step": round(b_ms, 4), "mean_context": round(b_ctx, 1), "hbm_gbs": round(b_gbs, 1),
                                    "hbm_frac": round(b_gbs / PEAK_HBM_GBS, 4), "frac_of_measured": round(b_gbs / read_gbs, 4)}
    for b in uneven:
        lengths = spread(b)
        v, b_ms, b_ctx = decode_run(b, max(20, args.steps // 2), max(4, args.warmup // 2), lengths)
        extra["decode_b%d_uneven" % b] = round(v, 1)
        b_gbs = (weight_bytes + b * b_ctx * kv_bytes_per_token) / (b_ms * 1e-3) / 1e9
        detail["decode_b%d_uneven" % b] = {"ms_per_step": round(b_ms, 4), "mean_context": round(b_ctx, 1), "longest_prompt": max(lengths),
                                           "shortest_prompt": min(lengths), "hbm_gbs": round(b_gbs, 1),
                                           "hbm_frac": round(b_gbs / PEAK_HBM_GBS, 4), "frac_of_measured": round(b_gbs / read_gbs, 4)}
    line = {
        "metric": "decode tok/s at batch %d (%s, %d-token prompts)" % (args.batch, shape_name, args.prompt_len),
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic (random weights, uniform-random token ids)",
        "config": {"model": shape_name, "layers": L, "layers_of_model": model_layers, "hidden": H, "q_heads": nq,
                   "kv_heads": nkv, "head_dim": d, "intermediate": I, "vocab": V, "global_batch": args.batch,
                   "seq_len": args.context, "prompt_len": args.prompt_len, "mean_context": round(ctx, 1), "page_size": page,
                   "graphs": not args.enforce_eager, "run_ahead": bool(eng.run_ahead), "parallelism": "single GPU",
                   "uneven_prompts": bool(args.spread), "keys_cut_by_host": bool(ops.DECODE_PIECES)},
        "prefill": {"value": round(T / pf, 1), "tokens": T, "ms": round(pf * 1e3, 3),
                    "frac": round(pf_flops / pf / PEAK_FLOPS[args.dtype], 4),
                    "library_tflops": None if lib_flops is None else round(lib_flops / 1e12, 1),
                    "frac_of_library": None if lib_flops is None else round(pf_flops / pf / lib_flops, 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4), "measured_read_gbs": round(read_gbs, 1),
                     "frac_of_measured": round(achieved / read_gbs, 4)},
        "points": extra,
        "points_detail": detail,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())

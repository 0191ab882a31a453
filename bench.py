"""Decode and prefill throughput of the engine at the Llama-3.2-1B shape, random weights, one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--config FILE] [--prefill-tokens T] [--layers L] [--no-points]
    python bench.py --fekorax [--sizes 1b,8b] [--layers L] [--batch B] [--prefill-tokens T]     (another record: see `fekorax_beside_llama`)
    python bench.py --rigalorn [--sizes 1b,8b] [--layers L] [--batch B] [--prefill-tokens T]    (another record: see `rigalorn_beside_fekorax`)
    python bench.py --zidevik [--sizes 1b,8b] [--layers L] [--batch B] [--prefill-tokens T]     (another record: see `zidevik_beside_rigalorn`)
    python bench.py --mimitar [--sizes 1b,8b] [--layers L] [--batch B] [--prefill-tokens T]     (another record: see `mimitar_beside_zidevik`)

A step is one decode step of the whole batch (default batch 8, each request on a 2,048-token
prompt in a 4,096-token context), through the scheduler with its defaults.  After W warm-up steps,
five windows of exactly K steps each are timed one after the other (5 K + W new tokens a request:
256 with the defaults, the benchmark's workload); `value` and `ms_per_step` are the median window's,
`ms_per_step_min` the fastest's.  Prints ONE JSON line: decoded tokens a second, the 2,048-token
prefill (median of 5), the decode step's roofline fraction against the published HBM peak and
against the read bandwidth a plain kernel of this library reaches on this chip, the prefill's
fraction against the published matrix peak and against a bare loop of matrix instructions, and decode
at batch 1 and 64 (medians of 5 windows as well).  --config FILE runs the same on another configuration of the
architecture (a config.json; `configs/` holds the Llama 3.2 3B and 3.1 8B shapes), --prefill-tokens T times a prompt of
another length.
"""
import argparse
import json
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

# MI355X published peaks
HBM_GBS = 8000.0
PEAK_TFLOPS = {"bf16": 2500.0, "fp32": 157.3}

LLAMA_1B = dict(hidden_size=2048, intermediate_size=8192, num_hidden_layers=16, num_attention_heads=32, num_key_value_heads=8,
                head_dim=64, vocab_size=128256, max_position_embeddings=4096, rope_theta=500000.0, rms_norm_eps=1e-5,
                tie_word_embeddings=True,
                rope_scaling=dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                  original_max_position_embeddings=8192))
PROMPT, NEW_TOKENS, CONTEXT, PAGE = 2048, 256, 4096, 16


# Layer shapes for `--fekorax`: (hidden, heads, key/value heads, head size, feed-forward's inner size, vocabulary).
FEKORAX_SIZES = {"1b": (2048, 32, 8, 64, 8192, 32000), "3b": (3072, 24, 8, 128, 8192, 32000), "8b": (4096, 32, 8, 128, 14336, 32000)}


def fekorax_beside_llama(args) -> int:
    """The Fekorax design at layer shapes of real models beside the Llama decoder at the same shapes, random weights: prefill of one
    prompt and decode steps of a batch on that context, through the step function (captured decode steps), and the time of every
    kernel in both (the device waited for around each).  A Fekorax model of L layers here is L/4 times [matrix memory; attention +
    feed-forward; matrix memory; attention on the pages of the one before + feed-forward], the attention with the Llama layer's
    heads (rotation of half of each head, chunks of 1,024, sinks, head gates), the matrix memories with a quarter as many heads of
    the same key size and twice the value size; the Llama model has L layers of attention + feed-forward.  One JSON line."""
    import torch
    from geneinfer_amd.config import parse_config
    from geneinfer_amd.engine import Runner, StepEntry, random_model
    from geneinfer_amd.kernels import ops

    T, batch, L, steps = args.prefill_tokens, args.batch, args.layers or 8, args.steps
    gen = torch.Generator().manual_seed(1)
    record = {"metric": "Fekorax beside Llama at equal layer shapes: prefill tok/s, decode ms a step, ms by kernel", "dtype": args.dtype, "layers": L,
              "prefill_tokens": T, "decode_batch": batch, "data": "synthetic: random weights by formula, uniform random token ids", "sizes": {}}
    for size in args.sizes.split(","):
        D, H, G, hd, ff, vocab = FEKORAX_SIZES[size]
        llama = dict(architectures=["LlamaForCausalLM"], hidden_size=D, intermediate_size=ff, num_hidden_layers=L, num_attention_heads=H,
                     num_key_value_heads=G, head_dim=hd, vocab_size=vocab, max_position_embeddings=T + 1024, rope_theta=500000.0, rms_norm_eps=1e-5,
                     tie_word_embeddings=True)
        att = lambda source=None: dict(type="attention", mlp=dict(kind="dense", ff=ff), mixer=dict(
            heads=H, kv_heads=G, dim=hd, vdim=hd, scale=hd ** -0.5, rot=dict(dims=hd // 2, base=10000.0), mask=dict(size=1024),
            **({} if source is None else dict(kv_from=source))))
        mem = dict(type="mlstm", mlp=None, mixer=dict(heads=max(1, H // 4), dim=hd, vdim=2 * hd, gate_cap=12.0))
        layers = []
        for i in range(0, L, 4):
            layers += [mem, att(), mem, att(i + 1)]
        fekorax = dict(architecture="Fekorax", vocab=vocab, width=D, embedding=dict(scale=D ** 0.5), norm=dict(eps=1e-5), layers=layers[:L],
                       max_positions=T + 1024)
        record["sizes"][size] = {}
        for name, cfg in (("llama", llama), ("fekorax", fekorax)):
            record["sizes"][size][name] = _measure_design(cfg, args, T, batch, steps, vocab, gen)
    print(json.dumps(record))
    return 0


def _measure_design(cfg, args, T, batch, steps, vocab, gen) -> dict:
    """Prefill of one prompt of T tokens (median over `batch` prompts), decode steps of the batch on those contexts (captured), and
    the time of every kernel in both (the device waited for around each)."""
    import torch
    from geneinfer_amd.config import parse_config
    from geneinfer_amd.engine import Runner, StepEntry, random_model
    from geneinfer_amd.kernels import ops
    model = random_model(parse_config(cfg), seed=0, dtype="bfloat16" if args.dtype == "bf16" else "float32", device="cuda:0", draw_on_device=True)
    runner = Runner(model, page_size=PAGE, max_tokens=batch * (T + 512), max_requests=batch, max_rows=max(T, batch), max_positions=T + 1024)
    prompts = [torch.randint(0, vocab, (T,), generator=gen).tolist() for _ in range(batch)]

    def prefill_all():
        times = []
        for r, p in enumerate(prompts):
            if runner.is_open(r):
                runner.close(r)
            runner.open(r)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            runner.step([StepEntry(r, p, (T - 1,))])
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
        return sorted(times)[len(times) // 2]

    def decode_steps(n):
        entries = [StepEntry(r, [7], (0,)) for r in range(batch)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            runner.step(entries)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / n

    prefill_all()
    prefill_s = prefill_all()
    decode_steps(args.warmup)
    decode_s = sorted(decode_steps(steps) for _ in range(3))[1]
    # the same once more with every kernel timed (no captured steps meanwhile)
    by_kernel = {}
    for what, run in (("prefill", lambda: (runner.close(0), runner.open(0), runner.step([StepEntry(0, prompts[0], (T - 1,))]))),
                      ("decode", lambda: decode_steps(4))):
        profile = ops.set_profiling(True)
        run()
        torch.cuda.synchronize()
        n = 1 if what == "prefill" else 4
        by_kernel[what] = {k: [profile.calls[k] // n, round(v * 1e3 / n, 4)] for k, v in sorted(profile.seconds.items(), key=lambda kv: -kv[1])}
        ops.set_profiling(False)
    result = {"prefill_tok_s": round(T / prefill_s, 1), "prefill_ms": round(prefill_s * 1e3, 3), "decode_ms_per_step": round(decode_s * 1e3, 4),
              "decode_tok_s": round(batch / decode_s, 1), "weight_bytes_per_step": model.weight_bytes_read_per_step(), "kernels_calls_ms": by_kernel}
    del runner, model
    torch.cuda.empty_cache()
    return result


def rigalorn_beside_fekorax(args) -> int:
    """The Rigalorn design at layer shapes of real models beside the Fekorax design (the nearest the engine has: memories and
    attention in turns) and the Llama decoder at the same shapes, random weights; measured as `fekorax_beside_llama` measures.  A
    Rigalorn model of L layers here is L/4 times [gated delta rule; attention through latents; attention with blended values;
    gated delta rule], every layer with its feed-forward beside the mixer: the attention with the Llama layer's heads (biases,
    rotation of half of each head with stretched frequencies, a window of 1,024), the latents of 4 and 12 head sizes for keys/values
    and queries with half a head size of rotated channels, the memories with a quarter as many heads of the same key size and twice
    the value size (as Fekorax's here), convolutions of 4 taps.  One JSON line."""
    import torch
    T, batch, L, steps = args.prefill_tokens, args.batch, args.layers or 8, args.steps
    gen = torch.Generator().manual_seed(1)
    record = {"metric": "Rigalorn beside Fekorax and Llama at equal layer shapes: prefill tok/s, decode ms a step, ms by kernel", "dtype": args.dtype, "layers": L,
              "prefill_tokens": T, "decode_batch": batch, "data": "synthetic: random weights by formula, uniform random token ids", "sizes": {}}
    for size in args.sizes.split(","):
        D, H, G, hd, ff, vocab = FEKORAX_SIZES[size]
        mlp = dict(kind="dense", ff=ff)
        llama = dict(architectures=["LlamaForCausalLM"], hidden_size=D, intermediate_size=ff, num_hidden_layers=L, num_attention_heads=H,
                     num_key_value_heads=G, head_dim=hd, vocab_size=vocab, max_position_embeddings=T + 1024, rope_theta=500000.0, rms_norm_eps=1e-5,
                     tie_word_embeddings=True)
        att = lambda source=None: dict(type="attention", mlp=mlp, mixer=dict(
            heads=H, kv_heads=G, dim=hd, vdim=hd, scale=hd ** -0.5, rot=dict(dims=hd // 2, base=10000.0), mask=dict(size=1024),
            **({} if source is None else dict(kv_from=source))))
        mem = dict(type="mlstm", mlp=None, mixer=dict(heads=max(1, H // 4), dim=hd, vdim=2 * hd, gate_cap=12.0))
        layers = []
        for i in range(0, L, 4):
            layers += [mem, att(), mem, att(i + 1)]
        fekorax = dict(architecture="Fekorax", vocab=vocab, width=D, embedding=dict(scale=D ** 0.5), norm=dict(eps=1e-5), layers=layers[:L], max_positions=T + 1024)
        delta = dict(type="delta", mlp=mlp, mixer=dict(heads=max(1, H // 4), kv_heads=max(1, H // 8), dim=hd, vdim=2 * hd, conv=4))
        latent = dict(type="latent_attention", mlp=mlp, mixer=dict(heads=H, dim=hd, rot_dim=hd // 2, vdim=hd, q_rank=12 * hd, kv_rank=4 * hd, scale=(1.5 * hd) ** -0.5,
                                                                    rot=dict(dims=hd // 2, base=500000.0), mask=dict(size=1024)))
        blended = dict(type="attention", mlp=mlp, mixer=dict(heads=H, kv_heads=G, dim=hd, vdim=hd, scale=hd ** -0.5, v_mix=True, mask=dict(size=1024), rot=dict(
            dims=hd // 2, base=10000.0, scaling=dict(factor=4.0, original=4096, fast=16.0, slow=2.0))))
        rigalorn = dict(architecture="Rigalorn", vocab=vocab, width=D, embedding=dict(scale=D ** 0.5), norm=dict(eps=1e-5), max_positions=T + 1024,
                        layers=([delta, latent, blended, delta] * ((L + 3) // 4))[:L])
        record["sizes"][size] = {}
        for name, cfg in (("llama", llama), ("fekorax", fekorax), ("rigalorn", rigalorn)):
            if args.only and name not in args.only.split(","):
                continue
            record["sizes"][size][name] = _measure_design(cfg, args, T, batch, steps, vocab, gen)
    print(json.dumps(record))
    return 0


def zidevik_beside_rigalorn(args) -> int:
    """The Zidevik design at layer shapes of real models beside the Rigalorn design (the nearest the engine has: parallel layers,
    attention and recurrences with short convolutions) and the Llama decoder at the same shapes, random weights; measured as
    `fekorax_beside_llama` measures.  Every Zidevik layer here has the Llama layer's attention heads (pairs of neighbours turned in
    half of each head, unit heads) beside a selective scan of twice the width with 16 states a channel, step sizes of rank width/16
    and 4 taps; the feed-forwards take turns: the Llama layer's dense one, then 8 experts of a quarter of its inner size, of which 2
    serve a token, with a shared expert of half of it (as many weights at work a token as the dense one).  Every layer reads 256
    columns of the tokens' second table.  Layers 0 and 1 are walked twice, so a model of L layers here runs L + 2.  The Rigalorn
    model is `rigalorn_beside_fekorax`'s.  One JSON line."""
    import torch
    T, batch, L, steps = args.prefill_tokens, args.batch, args.layers or 8, args.steps
    gen = torch.Generator().manual_seed(1)
    record = {"metric": "Zidevik beside Rigalorn and Llama at equal layer shapes: prefill tok/s, decode ms a step, ms by kernel", "dtype": args.dtype, "layers": L,
              "prefill_tokens": T, "decode_batch": batch, "data": "synthetic: random weights by formula, uniform random token ids", "sizes": {}}
    for size in args.sizes.split(","):
        D, H, G, hd, ff, vocab = FEKORAX_SIZES[size]
        mlp = dict(kind="dense", ff=ff)
        llama = dict(architectures=["LlamaForCausalLM"], hidden_size=D, intermediate_size=ff, num_hidden_layers=L, num_attention_heads=H,
                     num_key_value_heads=G, head_dim=hd, vocab_size=vocab, max_position_embeddings=T + 1024, rope_theta=500000.0, rms_norm_eps=1e-5,
                     tie_word_embeddings=True)
        delta = dict(type="delta", mlp=mlp, mixer=dict(heads=max(1, H // 4), kv_heads=max(1, H // 8), dim=hd, vdim=2 * hd, conv=4))
        latent = dict(type="latent_attention", mlp=mlp, mixer=dict(heads=H, dim=hd, rot_dim=hd // 2, vdim=hd, q_rank=12 * hd, kv_rank=4 * hd, scale=(1.5 * hd) ** -0.5,
                                                                    rot=dict(dims=hd // 2, base=500000.0), mask=dict(size=1024)))
        blended = dict(type="attention", mlp=mlp, mixer=dict(heads=H, kv_heads=G, dim=hd, vdim=hd, scale=hd ** -0.5, v_mix=True, mask=dict(size=1024), rot=dict(
            dims=hd // 2, base=10000.0, scaling=dict(factor=4.0, original=4096, fast=16.0, slow=2.0))))
        rigalorn = dict(architecture="Rigalorn", vocab=vocab, width=D, embedding=dict(scale=D ** 0.5), norm=dict(eps=1e-5), max_positions=T + 1024,
                        layers=([delta, latent, blended, delta] * ((L + 3) // 4))[:L])
        mixer = dict(left=dict(heads=H, kv_heads=G, dim=hd, vdim=hd, scale=hd ** -0.5, rot=dict(dims=hd // 2, base=500000.0)), left_scale=1.0,
                     right=dict(inner=2 * D, state=16, dt_rank=D // 16, conv=4), right_scale=1.0)
        moe = dict(kind="moe", router=dict(experts=8, top=2), expert=dict(ff=ff // 4), shared=dict(ff=ff // 2))
        zidevik = dict(architecture="Zidevik", vocab=vocab, width=D, norm=dict(eps=1e-5), max_positions=T + 1024, logit_softcap=30.0, token_side=dict(dim=256),
                       loop=dict(start=0, stop=min(2, L), times=2), layers=[dict(type="parallel", mixer=mixer, mlp=mlp if i % 2 == 0 else moe) for i in range(L)])
        record["sizes"][size] = {}
        for name, cfg in (("llama", llama), ("rigalorn", rigalorn), ("zidevik", zidevik)):
            if args.only and name not in args.only.split(","):
                continue
            record["sizes"][size][name] = _measure_design(cfg, args, T, batch, steps, vocab, gen)
    print(json.dumps(record))
    return 0


def mimitar_beside_zidevik(args) -> int:
    """The Mimitar design at layer shapes of real models beside the Zidevik design (the nearest the engine has: attention with a scale
    of its own and a rotation of a part of the head, routed experts with a shared one), the Rigalorn design (attention through
    latents) and the Llama decoder at the same shapes, random weights; measured as `fekorax_beside_llama` measures.  A Mimitar model
    of L layers here carries 4 copies of the residual stream; its layers take turns of four: attention with the Llama layer's heads
    (a norm over the whole query and key projections, a rotation of half of each head with stretched frequencies, scores capped at
    50) and the Llama layer's feed-forward with clamped halves; the same attention with 8 experts of a quarter of that inner size
    in 4 groups of which 2 are kept, 2 experts a token, and a gated shared expert of half of it; the first layer once more with its
    own cache (no weights of its own); attention through latents (Rigalorn's sizes, a gate per head) with the experts.  Every
    mixer's input is blended with the token before.  One JSON line."""
    import torch
    T, batch, L, steps = args.prefill_tokens, args.batch, args.layers or 8, args.steps
    gen = torch.Generator().manual_seed(1)
    record = {"metric": "Mimitar beside Zidevik, Rigalorn and Llama at equal layer shapes: prefill tok/s, decode ms a step, ms by kernel", "dtype": args.dtype, "layers": L,
              "prefill_tokens": T, "decode_batch": batch, "data": "synthetic: random weights by formula, uniform random token ids", "sizes": {}}
    for size in args.sizes.split(","):
        D, H, G, hd, ff, vocab = FEKORAX_SIZES[size]
        mlp = dict(kind="dense", ff=ff)
        llama = dict(architectures=["LlamaForCausalLM"], hidden_size=D, intermediate_size=ff, num_hidden_layers=L, num_attention_heads=H,
                     num_key_value_heads=G, head_dim=hd, vocab_size=vocab, max_position_embeddings=T + 1024, rope_theta=500000.0, rms_norm_eps=1e-5,
                     tie_word_embeddings=True)
        delta = dict(type="delta", mlp=mlp, mixer=dict(heads=max(1, H // 4), kv_heads=max(1, H // 8), dim=hd, vdim=2 * hd, conv=4))
        latent = dict(type="latent_attention", mlp=mlp, mixer=dict(heads=H, dim=hd, rot_dim=hd // 2, vdim=hd, q_rank=12 * hd, kv_rank=4 * hd, scale=(1.5 * hd) ** -0.5,
                                                                    rot=dict(dims=hd // 2, base=500000.0), mask=dict(size=1024)))
        blended = dict(type="attention", mlp=mlp, mixer=dict(heads=H, kv_heads=G, dim=hd, vdim=hd, scale=hd ** -0.5, v_mix=True, mask=dict(size=1024), rot=dict(
            dims=hd // 2, base=10000.0, scaling=dict(factor=4.0, original=4096, fast=16.0, slow=2.0))))
        rigalorn = dict(architecture="Rigalorn", vocab=vocab, width=D, embedding=dict(scale=D ** 0.5), norm=dict(eps=1e-5), max_positions=T + 1024,
                        layers=([delta, latent, blended, delta] * ((L + 3) // 4))[:L])
        mixer = dict(left=dict(heads=H, kv_heads=G, dim=hd, vdim=hd, scale=hd ** -0.5, rot=dict(dims=hd // 2, base=500000.0)), left_scale=1.0,
                     right=dict(inner=2 * D, state=16, dt_rank=D // 16, conv=4), right_scale=1.0)
        moe = dict(kind="moe", router=dict(experts=8, top=2), expert=dict(ff=ff // 4), shared=dict(ff=ff // 2))
        zidevik = dict(architecture="Zidevik", vocab=vocab, width=D, norm=dict(eps=1e-5), max_positions=T + 1024, logit_softcap=30.0, token_side=dict(dim=256),
                       loop=dict(start=0, stop=min(2, L), times=2), layers=[dict(type="parallel", mixer=mixer, mlp=mlp if i % 2 == 0 else moe) for i in range(L)])
        m_dense = dict(kind="dense", ff=ff, limit=7.0)
        m_moe = dict(kind="moe", router=dict(experts=8, top=2, groups=dict(count=4, keep=2)), expert=dict(ff=ff // 4, limit=7.0), shared=dict(ff=ff // 2, limit=7.0))
        m_att = dict(heads=H, kv_heads=G, dim=hd, vdim=hd, scale=hd ** -0.5, softcap=50.0,
                     rot=dict(dims=hd // 2, base=500000.0, scaling=dict(factor=32.0, low=1.0, high=4.0, original=8192)))
        m_latent = dict(heads=H, dim=hd, rot_dim=hd // 2, vdim=hd, q_rank=12 * hd, kv_rank=4 * hd, scale=(1.5 * hd) ** -0.5,
                        rot=dict(dims=hd // 2, base=500000.0, scaling=dict(factor=4.0, original=4096, fast=16.0, slow=2.0)))
        four = lambda i: [dict(type="attention", mixer=m_att, mlp=m_dense), dict(type="attention", mixer=m_att, mlp=m_moe),
                          dict(type="attention", mixer=m_att, mlp=m_dense, weights_of=i), dict(type="latent_attention", mixer=m_latent, mlp=m_moe)]
        mimitar = dict(architecture="Mimitar", vocab=vocab, width=D, norm=dict(eps=1e-5), streams=4, residual_mult=0.5, logit_scale=0.25, max_positions=T + 1024,
                       layers=[l for i in range(0, L, 4) for l in four(i)][:L])
        record["sizes"][size] = {}
        for name, cfg in (("llama", llama), ("rigalorn", rigalorn), ("zidevik", zidevik), ("mimitar", mimitar)):
            if args.only and name not in args.only.split(","):
                continue
            record["sizes"][size][name] = _measure_design(cfg, args, T, batch, steps, vocab, gen)
    print(json.dumps(record))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=48, help="decode steps per timed window (five windows are timed)")
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--dtype", choices=["bf16", "fp32"], default="bf16")
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the configuration has (0 = all); named in the record")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and batch 64 points")
    ap.add_argument("--config", default="", help="a config.json of another size of the architecture (default: the Llama-3.2-1B shape)")
    ap.add_argument("--prefill-tokens", type=int, default=PROMPT, help="length of the timed prompt")
    ap.add_argument("--fekorax", action="store_true", help="another measurement: the Fekorax design beside Llama at equal layer shapes (see fekorax_beside_llama)")
    ap.add_argument("--rigalorn", action="store_true", help="another measurement: the Rigalorn design beside Fekorax and Llama at equal layer shapes (see rigalorn_beside_fekorax)")
    ap.add_argument("--zidevik", action="store_true", help="another measurement: the Zidevik design beside Rigalorn and Llama at equal layer shapes (see zidevik_beside_rigalorn)")
    ap.add_argument("--mimitar", action="store_true", help="another measurement: the Mimitar design beside Zidevik, Rigalorn and Llama at equal layer shapes (see mimitar_beside_zidevik)")
    ap.add_argument("--only", default="", help="with --rigalorn, --zidevik or --mimitar: the designs to measure, of llama, fekorax, rigalorn, zidevik, mimitar (default: all)")
    ap.add_argument("--sizes", default="1b,8b", help="with --fekorax, --rigalorn, --zidevik or --mimitar: layer shapes, of " + ", ".join(FEKORAX_SIZES))
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this single-GPU engine")
        return 2

    if args.fekorax:
        return fekorax_beside_llama(args)
    if args.rigalorn:
        return rigalorn_beside_fekorax(args)
    if args.zidevik:
        return zidevik_beside_rigalorn(args)
    if args.mimitar:
        return mimitar_beside_zidevik(args)

    import torch
    from geneinfer_amd.config import LlamaConfig
    from geneinfer_amd.engine import Engine, EngineConfig, EngineRequest, Runner, StepEntry, random_model
    from geneinfer_amd.kernels import ops
    from geneinfer_amd.sampling import Sampler, SamplerConfig, sample_rows

    sizes, name = dict(LLAMA_1B), "Llama-3.2-1B"
    if args.config:
        sizes, name = json.loads(Path(args.config).read_text()), Path(args.config).stem
    T = args.prefill_tokens
    context_len = max(CONTEXT, T + 64)
    sizes["max_position_embeddings"] = max(context_len, sizes.get("max_position_embeddings", 0))
    layers_full = sizes["num_hidden_layers"]
    if args.layers:
        sizes["num_hidden_layers"] = args.layers
    config = LlamaConfig.from_dict(sizes) if not args.config else __import__("geneinfer_amd.config", fromlist=["parse_config"]).parse_config(sizes)
    dtype = "bfloat16" if args.dtype == "bf16" else "float32"
    model = random_model(config, seed=0, dtype=dtype, device="cuda:0", draw_on_device=True)
    vocab = config.vocab_size
    gen = torch.Generator().manual_seed(1)

    WINDOWS, PREFILL_WARMUP = 5, 4

    def make_runner(batch, per_request=0):
        per_request = per_request or -(-(PROMPT + WINDOWS * args.steps + args.warmup + 2 * batch + 8) // 64) * 64
        return Runner(model, page_size=PAGE, max_tokens=batch * per_request, max_requests=batch, max_rows=max(PROMPT, T, batch),
                      max_positions=context_len)

    def prefill(runner, rid, toks):
        runner.open(rid)
        return runner.step([StepEntry(rid, toks, (T - 1,))])

    def decode(batch, steps, warmup):
        """Greedy decoding of `batch` requests after their prompts, through the scheduler as serving runs it (its
        defaults: prefix sharing on, decoding ahead); returns [(seconds for `steps` decode steps, mean context at the
        middle of them)] for WINDOWS windows timed one after the other, sorted by time."""
        runner = make_runner(batch)
        engine = Engine(runner, EngineConfig(max_running=batch))
        limit = min(CONTEXT, PROMPT + WINDOWS * steps + warmup + 2 * batch + 4)
        for r in range(batch):
            engine.submit(EngineRequest(torch.randint(0, vocab, (PROMPT,), generator=gen).tolist(), limit, SamplerConfig(temperature=0.0)))
        decoding = 0
        while decoding < 2:                                  # the prompts, in steps of up to max_rows rows, until steps hold decode rows only
            rows = engine.stats.rows
            assert engine.step()
            decoding = decoding + 1 if engine.stats.rows - rows == batch and engine.stats.passes > batch else 0
        for _ in range(warmup):
            engine.step()
        windows = []
        for _ in range(WINDOWS):
            torch.cuda.synchronize()
            context = sum(runner.length(job.key) for job in engine.running) / batch + steps / 2
            passes = engine.stats.passes
            t0 = time.perf_counter()
            for _ in range(steps):
                engine.step()
            torch.cuda.synchronize()
            windows.append((time.perf_counter() - t0, context))
            assert engine.stats.passes - passes == steps and len(engine.running) == batch, "a timed step was not a decode step of the whole batch"
        del engine, runner
        torch.cuda.empty_cache()
        return sorted(windows)

    # ---- prefill of one 2,048-token prompt (median of 5 after PREFILL_WARMUP untimed ones: the first few run some percent slower)
    runner = make_runner(1, T + 64)
    greedy = Sampler(SamplerConfig(temperature=0.0), vocab)
    times = []
    for i in range(PREFILL_WARMUP + 5):
        toks = torch.randint(0, vocab, (T,), generator=gen).tolist()            # the prompt is there before the clock starts
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        logits = prefill(runner, i, toks)
        sample_rows(logits, [greedy])          # the first token reaches the host, drawn as generation draws it
        times.append(time.perf_counter() - t0)
        runner.close(i)
    prefill_s = sorted(times[PREFILL_WARMUP:])[2]
    del runner
    torch.cuda.empty_cache()
    L, D, I, V = config.num_hidden_layers, config.hidden_size, config.intermediate_size, vocab
    A, KV, hd, H = config.attn_dim, config.kv_dim, config.head_dim, config.num_attention_heads
    layer_params = D * (A + 2 * KV) + A * D + 3 * I * D
    prefill_flops = 2.0 * L * layer_params * T + L * 4.0 * H * hd * T * (T + 1) / 2 + 2.0 * V * D
    prefill_rec = {"value": round(T / prefill_s, 1), "tokens": T, "ms": round(prefill_s * 1e3, 3),
                   "frac": round(prefill_flops / prefill_s / (PEAK_TFLOPS[args.dtype] * 1e12), 4)}

    # ---- what a plain kernel reads and a bare loop of matrix instructions computes on this chip
    own_gbs = ops.measured_read_bandwidth("cuda:0")
    own_tflops = ops.measured_mfma_rate("cuda:0") if args.dtype == "bf16" else None
    prefill_rec["tflops"] = round(prefill_flops / prefill_s / 1e12, 1)
    if own_tflops:
        prefill_rec["own_peak_tflops"], prefill_rec["frac_of_own_peak"] = round(own_tflops, 1), round(prefill_flops / prefill_s / 1e12 / own_tflops, 4)

    # ---- decode
    windows = decode(args.batch, args.steps, args.warmup)
    dt, context = windows[len(windows) // 2]
    elem = 2 if args.dtype == "bf16" else 4
    weight_bytes = model.weight_bytes_read_per_step()
    kv_bytes = args.batch * context * L * 2 * KV * elem
    achieved = (weight_bytes + kv_bytes) / (dt / args.steps) / 1e9
    points = {}
    if not args.no_points:
        for b in (1, 64):
            w = decode(b, max(8, args.steps // 2), 8)
            points[f"decode_b{b}"] = round(b * max(8, args.steps // 2) / w[len(w) // 2][0], 1)

    rec = {
        "metric": f"decode tok/s at batch 1/8/64 + prefill tok/s at {T:,} tokens, {name}",
        "value": round(args.batch * args.steps / dt, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(dt / args.steps * 1e3, 4), "ms_per_step_min": round(windows[0][0] / args.steps * 1e3, 4), "windows": WINDOWS,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic: random weights N(0, 0.02) by a stated formula of seed, tensor name and index, uniform random token ids",
        "config": {"model": f"{name} shape", "layers": L, "layers_of_config": layers_full, "hidden": D, "heads": H,
                   "kv_heads": config.num_key_value_heads, "head_dim": hd, "intermediate": I, "vocab": V, "global_batch": args.batch,
                   "seq_len": context_len, "prompt_len": PROMPT, "decode_context": context, "page_size": PAGE, "tied_embeddings": bool(sizes.get("tie_word_embeddings", False)),
                   "rope": f"{(sizes.get('rope_scaling') or {}).get('rope_type', 'plain')} theta {sizes.get('rope_theta', 10000.0):g} factor {(sizes.get('rope_scaling') or {}).get('factor', 1):g}",
                   "parallelism": "single_gpu"},
        "prefill": prefill_rec,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBS, "unit": "GB/s", "frac": round(achieved / HBM_GBS, 4),
                     "own_peak": round(own_gbs, 1), "frac_of_own_peak": round(achieved / own_gbs, 4)},
        "points": points,
    }
    print(json.dumps(rec))
    return 0


if __name__ == "__main__":
    sys.exit(main())

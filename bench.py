#!/usr/bin/env python3
"""Decode benchmark: Llama2-7B-shape INT4 greedy decode on one MI355X.

A "step" is one iteration of the decode loop (one new token per sequence): embedding, 32
transformer blocks (RMSNorm, INT4 q/k/v/o and SwiGLU projections, rotary embedding, KV append,
attention over the cache, residuals), final norm, fp16 lm_head, greedy selection and the loop
bookkeeping.  The default run follows the headline configuration: batch 1, a 128-token prompt, then
256 timed new tokens (contexts 128..383), KV cache length 2048.  The prompt's 128 loop iterations are
always run untimed first (in passes of up to 1024 rows; ``--prompt-loop``: one iteration per position, as
the reference's loop does), then ``--warmup`` further untimed iterations, then ``--steps`` timed ones: the
timed iterations generate new tokens whatever the flags are.

By default the iteration runs as one persistent launch (pta_llama_decode_step, batch <= 16);
``--executor operators`` runs it as one launch per operator instead.

The default run also measures batch 16 (same model, step counts and executor) and reports it under "batch16"
beside the batch-1 headline, and - bounded to a few seconds each - the other benchmark configurations under
"single_operator" (the INT4 operator at M = 1, 4, 16, 64), "chatglm2_fp8_b8", "rwkv_b1", "rwkv_b32" and
"gpt2_small" (``--no-extras`` skips them).  Progress lines go to stderr; the JSON line is the only stdout output.

Prints ONE JSON line with tokens/s, the HBM roofline of the dominant kernel measured with events
on the stream it runs on (the persistent decode-step kernel: one launch moves the whole step's
bytes; or, with the per-operator executor, the fused INT4 gate/up projection), and a CPU baseline
(the numpy restatement of the same graph on the host cores, on a reduced number of layers).

Other workloads (``--workload``), each printing one line of the same form: ``gemm`` = the single INT4
weight-only operator X[M, 4096] by W[4096, 11008] at M = ``--batch``; ``chatglm2`` = ChatGLM2-6B-shape FP8
decode; ``rwkv`` = RWKV-4-7B-shape INT4 recurrent decode; ``prompt`` = the prompt of the headline model taken in
passes of ``--rows-per-pass`` rows (a step is one pass) instead of one position per loop iteration.  ``--copy-calibration`` and ``--summarize-pmc``
serve the hardware-counter measurement of the HBM traffic (see their help).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

LLAMA2_7B = dict(vocab_size=32000, hidden_size=4096, rms_norm_eps=1e-5, num_attention_heads=32,
                 intermediate_size=11008, num_hidden_layers=32)
MAX_LEN = 2048
PROMPT = 128            # prompt positions of the headline configuration; always consumed untimed
HBM_PEAK_GBS = 8000.0
_T0 = time.perf_counter()


def note(msg):
    """Progress line on stderr (stdout carries the one JSON line): a run that is slow - under a profiler, say -
    can be told from one that hangs."""
    print("[bench %7.1fs] %s" % (time.perf_counter() - _T0, msg), file=sys.stderr, flush=True)


def run_steps_noted(dec, n, what, chunk=64):
    """dec.run_steps(n) in chunks, each followed by a synchronisation and a progress line.  Untimed phases only."""
    import torch
    done = 0
    while done < n:
        k = min(chunk, n - done)
        dec.run_steps(k)
        torch.cuda.synchronize()
        done += k
        note(f"{what}: {done}/{n} iterations")


def check_persistent(dec, what):
    """Exit at once, with the reason, when the persistent decode step has reported a failure."""
    if getattr(dec, "persistent", None) is not None and dec.persistent.failed():
        print(f"{what}: the persistent decode step reported a failure (a workgroup gave up waiting: the kernel needs every "
              "compute unit of the device for itself while it runs)", file=sys.stderr, flush=True)
        sys.exit(1)


def algorithmic_step_bytes(cfg, B, t, kv_bytes=2):
    """Bytes one decode step must move at context t: every weight once (INT4 + scales, norm
    weights, fp16 lm_head), the KV rows written and read (kv_bytes per element), the embedding rows."""
    d, f, v, n = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"], cfg["num_hidden_layers"]
    per_layer = (4 * d * d + 3 * d * f) // 2 + 2 * (4 * d + 2 * f + d)
    weights = n * per_layer + 2 * (2 * n + 1) * d + 2 * v * d
    kv = B * 2 * n * d * kv_bytes * (t + 1)
    return weights + kv + B * d * 2


def cpu_baseline(seconds_budget=20.0):
    """The numpy oracle of the same graph on the host: 2 full-width layers + head, scaled to 32."""
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    from oracle import models as OM
    try:
        from threadpoolctl import threadpool_info
        threads = max([p.get("num_threads", 1) for p in threadpool_info()] or [1])
    except Exception:
        threads = os.cpu_count() or 1
    layers = 2
    cfg = dict(LLAMA2_7B, num_hidden_layers=layers)
    sd = OM.make_llama2_state_dict(cfg, seed=0, int4=True)
    L = 64
    model = OM.Llama2Oracle(sd, cfg, L, 1)
    ids = np.zeros((1, L), np.int32)
    ids[0, :8] = np.arange(5, 13)
    from oracle import ops as O
    state = O.initial_loop_state(ids, L)
    model.step(state["container"][:, 0].reshape(1, 1), 0, state["mask"])       # warm-up
    n, t0 = 0, time.perf_counter()
    t_layers = t_head = 0.0
    while time.perf_counter() - t0 < seconds_budget and n < 12:
        step = n + 1
        a = time.perf_counter()
        x = model.embed[state["container"][:, step].reshape(1, 1)]
        mask4 = state["mask"][:, None, None, :]
        for lay in model.layers:
            t = O.rms_norm(x, lay["ln1"], model.eps)
            t = model._attention(lay, t, step, mask4)
            x = (x + t).astype(np.float16)
            t = O.rms_norm(x, lay["ln2"], model.eps).reshape(-1, model.d)
            u = (lay["up"](t) * O.swish(lay["gate"](t))).astype(np.float16)
            x = (x + lay["down"](u).reshape(1, -1, model.d)).astype(np.float16)
        b = time.perf_counter()
        O.topk1(model.head(O.rms_norm(x, model.norm, model.eps)), axis=2)
        c = time.perf_counter()
        t_layers += b - a
        t_head += c - b
        state["mask"][:, step + 1] = 0
        n += 1
    per_token = (t_layers / n) * (LLAMA2_7B["num_hidden_layers"] / layers) + t_head / n
    return {"value": 1.0 / per_token, "unit": "tokens/s", "cores": int(threads), "kind": "port",
            "sample": f"numpy oracle, {layers} full-width layers + lm_head, {n} tokens at batch 1, "
                      f"layer time scaled x{LLAMA2_7B['num_hidden_layers'] // layers}"}


def pmc_summary_path(B):
    """The committed hardware-counter summary of the decode-step kernel at batch B (1 and 16 are recorded)."""
    return os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", f"llama2_7b_int4_b{B}_decode_step_pmc.txt")


def summarize_pmc(fetch_csv, write_csv):
    """FETCH_SIZE / WRITE_SIZE (KiB per dispatch) of the decode-step kernel, each scaled by what the
    same counter reads for the 1 GiB calibration kernel of --copy-calibration."""
    import csv

    def per_kernel(path, counter):
        vals = {}
        for r in csv.DictReader(open(path)):
            if r["Counter_Name"] == counter:
                vals.setdefault(r["Kernel_Name"], []).append(float(r["Counter_Value"]))
        return vals

    out = {}
    for counter, path in (("FETCH_SIZE", fetch_csv), ("WRITE_SIZE", write_csv)):
        vals = per_kernel(path, counter)
        step = [v for k, v in vals.items() if "decode_step_kernel" in k or "decode_step_wide_kernel" in k]
        cal = [v for k, v in vals.items() if "neg_kernel" in k or "NegFunctor" in k or "neg" in k.lower()]
        if not step or not cal:
            raise SystemExit(f"{path}: decode-step or calibration kernel not found")
        step, cal = step[0], cal[0]
        cal_kib = sum(cal) / len(cal)
        factor = (1 << 20) / cal_kib                      # the calibration kernel moves 1 GiB = 2^20 KiB each way
        mean_kib = sum(step) / len(step)
        out[counter] = mean_kib * factor * 1024
        print(f"{counter}: decode-step kernel mean {mean_kib:.1f} KiB over {len(step)} launches "
              f"(min {min(step):.1f}, max {max(step):.1f}); calibration kernel reads {cal_kib:.1f} KiB for 2^20 KiB "
              f"-> factor {factor:.4f} -> {out[counter]:.0f} bytes per launch")
    print(f"traffic_bytes_per_launch = {out['FETCH_SIZE'] + out['WRITE_SIZE']:.0f}")


def recorded_traffic(B):
    """HBM bytes per launch of the decode-step kernel from the committed counter summary, or None."""
    try:
        for line in open(pmc_summary_path(B)):
            if line.startswith("traffic_bytes_per_launch"):
                return float(line.split("=")[1])
    except OSError:
        pass
    return None


def gemm_measure(M, steps, warmup, weights=None):
    """Single-operator INT4 weight-only GEMV/GEMM: X[M, 4096] fp16 by W[4096, 11008] packed INT4 with
    per-output-channel fp16 scales -> fp16 [M, 11008].  A step is one launch; 48 copies of the weight
    (1 GiB in all) are used in turn so that no launch finds its weight in a cache.  Returns the result dict and
    the weight copies (so that several M share them)."""
    import torch
    from poptransformer_amd import kernels as K
    Kd, N, copies = 4096, 11008, 48
    gen = torch.Generator(device="cuda").manual_seed(7)
    x = torch.randn(M, Kd, device="cuda", dtype=torch.float16, generator=gen)
    ws = weights
    if ws is None:
        ws = []
        for _ in range(copies):
            packed = torch.randint(0, 256, (N, Kd // 2), device="cuda", dtype=torch.uint8, generator=gen).view(torch.int8)
            scale = (torch.rand(N, device="cuda", generator=gen) * 0.015 + 0.005).to(torch.float16)
            ws.append(K.W4Weight(packed, scale))
            del packed
    out = torch.empty(M, N, device="cuda", dtype=torch.float16)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for w in ws:
            K.w4a16_gemm(x, w, out=out)
        stream.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=stream):
            for w in ws:
                K.w4a16_gemm(x, w, out=out)
        rounds_w = max(1, warmup // copies)
        rounds = max(1, steps // copies)
        for _ in range(rounds_w):
            g.replay()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(rounds):
            g.replay()
        e1.record(stream)
    torch.cuda.synchronize()
    n = rounds * copies
    sec = e0.elapsed_time(e1) * 1e-3 / n
    nbytes = Kd * N // 2 + 2 * N + 2 * M * Kd + 2 * M * N
    achieved = nbytes / sec / 1e9
    return {"M": M, "launches": n, "warmup": rounds_w * copies, "us_per_launch": sec * 1e6, "bytes_per_launch": nbytes,
            "achieved_gbs": achieved, "frac": achieved / HBM_PEAK_GBS, "tflops": 2.0 * M * Kd * N / sec / 1e12}, ws


def gemm_workload(args):
    M = args.batch
    r, _ = gemm_measure(M, args.steps, args.warmup)
    return {
        "metric": "INT4 weight-only GEMV/GEMM launches/s", "value": 1e6 / r["us_per_launch"], "unit": "launches/s", "n_gpus": 1,
        "steps": r["launches"], "warmup": r["warmup"], "ms_per_step": r["us_per_launch"] * 1e-3, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "int4 weights, f16 activations, f32 accumulation", "data": "synthetic",
        "config": {"workload": f"single-operator W4A16: X[{M},4096] fp16 by W[4096,11008] packed INT4, fp16 scales", "M": M},
        "roofline": {"bound": "hbm", "kernel": "pta_w4a16_gemm", "achieved": r["achieved_gbs"], "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": r["frac"], "traffic": None, "bytes_per_launch": r["bytes_per_launch"],
                     "avg_launch_us": r["us_per_launch"], "tflops": r["tflops"]},
    }



CHATGLM2_6B = dict(num_layers=28, hidden_size=4096, num_attention_heads=32, multi_query_group_num=2, ffn_hidden_size=13696,
                   padded_vocab_size=65024, layernorm_epsilon=1e-5)
RWKV4_7B = dict(num_hidden_layers=32, hidden_size=4096, attention_hidden_size=4096, intermediate_size=16384,
                vocab_size=65536, layer_norm_epsilon=1e-5, rescale_every=6)


def other_model_workload(workload, B, steps, warmup, prompt_loop=False):
    """ChatGLM2-6B-shape FP8 decode (F143 weights and activations, fp16 KV cache of length 4096) or
    RWKV-4-7B-shape INT4 recurrent decode, one launch per operator replayed from a HIP graph.  The prompt of
    the configuration (512 / 64 positions) is consumed untimed, then `warmup` further untimed iterations.
    Reported like the headline, without a kernel leg."""
    import torch
    from poptransformer_amd.engine import fused, loader, rwkv, synthetic
    rng = np.random.Generator(np.random.PCG64(1234))
    prompt = 512 if workload == "chatglm2" else 64          # of the respective benchmark configuration
    first = prompt + warmup                                  # first timed loop iteration
    note(f"{workload} batch {B}: generating weights")
    if workload == "chatglm2":
        cfg, max_len = CHATGLM2_6B, 4096
        weights = synthetic.chatglm2_synthetic_weights(cfg, "fp8", seed=0)
        dec = fused.FusedDecoder(loader.chatglm2_spec(cfg, max_len, B, pad_id=0, eos_id=2), weights)
        hd = cfg["hidden_size"] // cfg["num_attention_heads"]
        per_pos = B * cfg["num_layers"] * 2 * cfg["multi_query_group_num"] * hd * 2
        wbytes, vocab = weights.nbytes(), cfg["padded_vocab_size"]
        name = "ChatGLM2-6B-shape FP8 (F143 weights and activations, F143 lm_head) greedy decode"
        dtype = "fp8 (F143) weights and activations decoded to f16, f32 accumulation"

        def step_bytes(t):
            return wbytes + per_pos * (t + 1) + B * cfg["hidden_size"] * 2
    else:
        cfg, max_len = RWKV4_7B, first + steps + 2
        weights = synthetic.rwkv_synthetic_weights(cfg, seed=0)
        dec = rwkv.RWKVDecoder(loader.rwkv_spec(cfg, max_len, B, pad_id=0, eos_id=-1), weights)
        wbytes, vocab = weights.nbytes(), cfg["vocab_size"]
        state = B * 2 * cfg["num_hidden_layers"] * (2 * 2 + 3 * 4) * cfg["hidden_size"]
        name = "RWKV-4-7B-shape INT4 recurrent decode"
        dtype = "int4 weights, f16 activations, f32 accumulation and WKV state"

        def step_bytes(t):
            return wbytes + state + B * cfg["hidden_size"] * 2
    if first + steps + 1 > max_len:
        print(f"prompt ({prompt}) + warmup + steps must stay below the sequence length {max_len}", file=sys.stderr)
        sys.exit(2)
    dec.capture()
    ids = np.zeros((B, max_len), np.int32)
    ids[:, :prompt] = rng.integers(3, vocab, size=(B, prompt))
    dec.reset(ids)
    done = dec.consume_prompt(dec.prompt_positions()) if hasattr(dec, "consume_prompt") and not prompt_loop else 0
    note(f"{workload} batch {B}: prompt ({done} positions in passes), {first - done} untimed iterations")
    run_steps_noted(dec, first - done, f"{workload} batch {B} untimed")
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    dec.run_steps(steps)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    note(f"{workload} batch {B}: {steps} timed iterations, {dt / steps * 1e3:.3f} ms each")
    mean_bytes = float(np.mean([step_bytes(t) for t in range(first, first + steps)]))
    return {
        "metric": "decode tokens/s + % of HBM roofline", "value": B * steps / dt, "unit": "tokens/s", "n_gpus": 1,
        "steps": steps, "warmup": warmup, "ms_per_step": dt / steps * 1e3, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": dtype, "data": "synthetic",
        "config": {"workload": f"{name}, batch {B}, prompt {prompt} consumed "
                               f"{'in passes of up to 1024 rows' if done else 'token by token'} (untimed), timed context "
                               f"{first}..{first + steps - 1}", "batch": B, "executor": "operators"},
        "step_algorithmic_bytes": mean_bytes,
        "step_roofline_frac": mean_bytes / (dt / steps) / (HBM_PEAK_GBS * 1e9),
    }


def brief(r):
    """The figures of a full result line that go under a key of the headline's line."""
    return {"value": r["value"], "unit": r["unit"], "ms_per_step": r["ms_per_step"], "steps": r["steps"],
            "workload": r["config"]["workload"], "step_algorithmic_bytes": r["step_algorithmic_bytes"],
            "step_roofline_frac": r["step_roofline_frac"]}


GPT2_SMALL = dict(vocab_size=50257, n_embd=768, n_head=12, n_layer=12, n_positions=1024, layer_norm_epsilon=1e-5)


def gpt2_small_workload(cpu=True):
    """GPT-2 small fp16 greedy decode, batch 1, prompt 16, 32 new tokens, KV length 128 (the plumbing configuration):
    the decode loop on the GPU (one launch per operator, HIP graph) and - the configuration's CPU reference path -
    the numpy oracle of the same graph on the host cores, with the generated tokens compared."""
    import torch
    from poptransformer_amd.engine import fused, loader, synthetic
    cfg, L, B, prompt, new = GPT2_SMALL, 128, 1, 16, 32
    pad, eos = 50257 - 1, 50257 - 2          # ids the random prompt avoids
    note("gpt2 small: generating weights")
    sd = synthetic.gpt2_synthetic_state_dict(cfg, seed=0)
    dec = fused.FusedDecoder(loader.gpt2_spec(cfg, L, B, pad, eos), loader.gpt2_weights(sd, cfg))
    dec.capture()
    rng = np.random.Generator(np.random.PCG64(1234))
    ids = np.full((B, L), pad, np.int32)
    ids[:, :prompt] = rng.integers(0, eos, size=(B, prompt))
    dec.reset(ids)
    dec.run_steps(prompt)                     # the prompt's iterations, one position each, untimed
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    dec.run_steps(new)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    got = dec.container.cpu().numpy()
    wbytes = sum(int(np.prod(v.shape)) * 2 for k, v in sd.items() if "wpe" not in k)
    out = {"value": B * new / dt, "unit": "tokens/s", "ms_per_step": dt / new * 1e3, "steps": new,
           "workload": f"GPT-2 small fp16 greedy decode, batch 1, prompt {prompt} (untimed, token by token), {new} new tokens, "
                       f"KV cache of {L}", "executor": "operators",
           "step_algorithmic_bytes": float(wbytes), "step_roofline_frac": wbytes / (dt / new) / (HBM_PEAK_GBS * 1e9)}
    note(f"gpt2 small: {dt / new * 1e3:.3f} ms per token on the GPU")
    if cpu:
        from oracle import models as OM
        try:
            from threadpoolctl import threadpool_info
            threads = max([p.get("num_threads", 1) for p in threadpool_info()] or [1])
        except Exception:
            threads = os.cpu_count() or 1
        model = OM.GPT2Oracle(sd, cfg, L, B)
        trace = []
        t0 = time.perf_counter()
        ref, _ = OM.run_decode_loop(model, ids, L, prompt + new, pad, eos, trace=trace)
        cdt = time.perf_counter() - t0
        out["cpu_baseline"] = {"value": B * (prompt + new) / cdt, "unit": "tokens/s", "cores": int(threads), "kind": "port",
                               "sample": f"numpy oracle of the same graph, all 12 layers, {prompt + new} loop iterations at batch 1"}
        ref = np.asarray(ref)
        same = ref[0, :prompt + new + 1] == got[0, :prompt + new + 1]
        out["tokens_equal_cpu"] = bool(same.all())
        if not same.all():
            # random N(0, 0.02) weights give nearly flat logits: say how close the oracle's two best were where the
            # generations part (iteration i selects the token of position i + 1)
            at = int(np.argmin(same))
            top2 = np.sort(trace[at - 1][1][0].astype(np.float64))[-2:]
            out["first_difference"] = {"position": at, "new_tokens_equal_before": max(0, at - prompt),
                                       "oracle_top2_gap_rel": float((top2[1] - top2[0]) / np.abs(trace[at - 1][1]).max())}
        note(f"gpt2 small: {cdt / (prompt + new) * 1e3:.1f} ms per token on the host, tokens equal: {out['tokens_equal_cpu']}")
    return out


def prompt_workload(args):
    """The prompt of the Llama2-7B-shape INT4 model in passes (FusedDecoder.consume_prompt): a step is one pass of
    --rows-per-pass // batch consecutive positions of every sequence through the 32 blocks (no head: the loop discards the
    tokens of these positions).  --steps passes are timed after one untimed run of the same prompt; the number of
    passes is capped by the KV cache length."""
    import torch
    from poptransformer_amd.engine import fused, loader, synthetic
    B, cfg = args.batch, LLAMA2_7B
    rows = args.rows_per_pass
    if B > rows or rows > 2048:
        print("the prompt passes take at most 2048 rows: batch <= --rows-per-pass <= 2048", file=sys.stderr)
        sys.exit(2)
    R = rows // B
    passes = max(1, min(args.steps, (MAX_LEN - 2) // R))
    n = passes * R
    weights = synthetic.llama2_synthetic_weights(cfg, seed=0)
    dec = fused.FusedDecoder(loader.llama2_spec(cfg, MAX_LEN, B, pad_id=0, eos_id=2, fp8_cache=args.fp8_cache), weights)
    rng = np.random.Generator(np.random.PCG64(1234))
    ids = np.zeros((B, MAX_LEN), np.int32)
    ids[:, :n + 1] = rng.integers(3, cfg["vocab_size"], size=(B, n + 1))
    dec.reset(ids)
    dec.consume_prompt(n, rows_per_pass=R)     # untimed: allocates the row buffers, warms every code path
    dec.reset(ids)
    dec.consume_prompt(n, rows_per_pass=R)     # untimed: records the pass into a HIP graph
    dec.reset(ids)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    dec.consume_prompt(n, rows_per_pass=R)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    d, f, nl = cfg["hidden_size"], cfg["intermediate_size"], cfg["num_hidden_layers"]
    per_layer = (4 * d * d + 3 * d * f) // 2 + 2 * (4 * d + 2 * f + d) + 2 * 2 * d
    # per pass: every block's weights once, the pass's K/V rows written, the cache read once per sequence
    kvb = 1 if args.fp8_cache else 2          # bytes per cache element
    kv = float(np.mean([B * nl * 2 * d * kvb * (p * R + R) + B * nl * 2 * d * kvb * R for p in range(passes)]))
    pass_bytes = nl * per_layer + kv + 2 * B * R * d
    flops = 2.0 * B * R * nl * (4 * d * d + 3 * d * f)
    return {
        "metric": "prompt tokens/s", "value": B * n / dt, "unit": "tokens/s", "n_gpus": 1, "steps": passes, "warmup": passes,
        "ms_per_step": dt / passes * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int4 weights, f16 activations, f32 accumulation", "data": "synthetic",
        "config": {"workload": f"Llama2-7B-shape INT4 prompt of {n} positions per sequence in {passes} passes of {R} positions, "
                               f"batch {B}, {'F143' if args.fp8_cache else 'fp16'} KV cache of {MAX_LEN}", "batch": B, "rows_per_pass": B * R,
                   "executor": "operators"},
        "step_algorithmic_bytes": pass_bytes,
        "step_roofline_frac": pass_bytes / (dt / passes) / (HBM_PEAK_GBS * 1e9),
        "projection_tflops": flops / (dt / passes) / 1e12,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=0,
                    help="decode workload: untimed loop iterations AFTER the 128-token prompt (which is always consumed "
                         "untimed); other workloads: untimed steps")
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--executor", choices=["persistent", "operators"], default=None,
                    help="default: persistent when the batch fits it (<= 16, fp16 cache), else operators")
    ap.add_argument("--workload", choices=["decode", "gemm", "chatglm2", "rwkv", "prompt"], default="decode",
                    help="decode: the Llama2-7B-shape INT4 decode loop (the headline); gemm: the single INT4 "
                         "weight-only operator at M = --batch rows; chatglm2: ChatGLM2-6B-shape FP8 decode; "
                         "rwkv: RWKV-4-7B-shape INT4 recurrent decode; prompt: the headline model's prompt in passes "
                         "of --rows-per-pass rows (--steps passes)")
    ap.add_argument("--rows-per-pass", type=int, default=64,
                    help="prompt workload: rows (batch x positions) per pass, up to 2048")
    ap.add_argument("--fp8-cache", action="store_true",
                    help="decode workload, operators executor: keep the KV cache as F143 bytes (KVCacheOp with fp8 = true)")
    ap.add_argument("--fuse-norm", choices=["on", "off"], default=None,
                    help="operators executor: run the norms inside the projections that consume them (default: the decoder's choice)")
    ap.add_argument("--prompt-loop", action="store_true",
                    help="decode workload: consume the (untimed) prompt one loop iteration per position, as the reference's "
                         "loop does, instead of in passes of up to 1024 rows (FusedDecoder.consume_prompt)")
    ap.add_argument("--no-batch16", action="store_true",
                    help="default run only: skip the second, batch-16 measurement that is reported beside the headline")
    ap.add_argument("--no-extras", action="store_true",
                    help="default run only: skip the other benchmark configurations (single operator, ChatGLM2, RWKV, GPT-2 small) "
                         "that are reported under keys of their own")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain elementwise kernel over 1 GiB three times (reads 1 GiB, writes 1 GiB): a kernel "
                         "of known traffic for scaling hardware counters (FETCH_SIZE / WRITE_SIZE) collected over this run")
    ap.add_argument("--summarize-pmc", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"),
                    help="no GPU work: print the traffic summary of two rocprofv3 --pmc runs of this script "
                         "(counter_collection.csv of the FETCH_SIZE run and of the WRITE_SIZE run, both with --copy-calibration)")
    args = ap.parse_args()
    if args.summarize_pmc:
        summarize_pmc(*args.summarize_pmc)
        return
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    if args.workload == "decode" and PROMPT + args.warmup + args.steps + 1 > MAX_LEN:
        print(f"prompt ({PROMPT}) + warmup + steps must stay below the KV cache length {MAX_LEN}", file=sys.stderr)
        sys.exit(2)

    import torch
    from poptransformer_amd import kernels as K
    from poptransformer_amd.engine import fused, loader, synthetic

    if not torch.cuda.is_available():
        print("no GPU visible", file=sys.stderr)
        sys.exit(1)
    if args.workload == "gemm":
        print(json.dumps(gemm_workload(args)))
        return
    if args.workload in ("chatglm2", "rwkv"):
        print(json.dumps(other_model_workload(args.workload, args.batch, args.steps, args.warmup, args.prompt_loop)))
        return
    if args.workload == "prompt":
        print(json.dumps(prompt_workload(args)))
        return
    B, cfg = args.batch, LLAMA2_7B
    executor = args.executor or ("persistent" if B <= 16 else "operators")
    kvb = 1 if args.fp8_cache else 2          # bytes per KV cache element
    note("generating the Llama2-7B-shape INT4 weights on the device")
    weights = synthetic.llama2_synthetic_weights(cfg, seed=0)
    rng = np.random.Generator(np.random.PCG64(1234))
    prompt = PROMPT
    t_first = prompt + args.warmup

    def decoder(batch):
        d = fused.FusedDecoder(loader.llama2_spec(cfg, MAX_LEN, batch, pad_id=0, eos_id=2, fp8_cache=args.fp8_cache), weights)
        if args.fuse_norm is not None:
            d.fuse_norm = args.fuse_norm == "on"
        if executor == "persistent":
            d.enable_persistent()
        d.capture()                       # one eager iteration, then the recording of one
        torch.cuda.synchronize()
        check_persistent(d, f"batch {batch}, first launches")
        note(f"batch {batch}: decoder ready ({executor}), first launches completed")
        return d

    def timed_decode(d, batch):
        """The prompt's 128 loop iterations untimed (contexts 0..127; in passes of up to 1024 rows unless
        --prompt-loop), then --warmup further iterations, then --steps timed ones: whatever --warmup is, the timed
        iterations start at context 128 + warmup and generate new tokens.  Wall clock around the timed iterations,
        and events around the same launches on the stream they are launched on."""
        ids = np.zeros((batch, MAX_LEN), np.int32)                       # pad id 0 after the prompt
        ids[:, :prompt] = rng.integers(3, cfg["vocab_size"], size=(batch, prompt))
        d.reset(ids)
        done = 0 if args.prompt_loop else d.consume_prompt(d.prompt_positions())
        note(f"batch {batch}: prompt consumed ({'in one pass' if done else 'token by token'})")
        run_steps_noted(d, prompt - done + args.warmup, f"batch {batch} untimed")
        check_persistent(d, f"batch {batch}, untimed iterations")
        cur = torch.cuda.current_stream()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0.record(cur)
        d.run_steps(args.steps)
        e1.record(cur)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        check_persistent(d, f"batch {batch}, timed iterations")
        note(f"batch {batch}: {args.steps} timed iterations, {dt / args.steps * 1e3:.4f} ms each")
        mean_bytes = float(np.mean([algorithmic_step_bytes(cfg, batch, t, kvb) for t in range(t_first, t_first + args.steps)]))
        return dt, e0.elapsed_time(e1) * 1e-3, mean_bytes, done

    def step_kernel_name(batch):
        kv8 = "true" if args.fp8_cache else "false"      # the kernels' last template argument: FP8 KV rings
        return ("decode_step_kernel<2, 6, 3, %d, %s>" % (1 if batch == 1 else 4, kv8) if batch <= 4 else
                "decode_step_wide_kernel<2, 6, 3, %s>" % kv8) + " (whole decode step)"

    def traffic_fields(batch):
        t = recorded_traffic(batch) if executor == "persistent" and not args.fp8_cache else None
        return {"traffic": t,
                "traffic_source": ("recorded, not measured in this run: hardware counters of an earlier profiled run, "
                                   "profiles/" + os.path.basename(pmc_summary_path(batch))) if t is not None else None}

    dec = decoder(B)
    dt, ev_s, mean_bytes, in_passes = timed_decode(dec, B)
    ms_per_step = dt / args.steps * 1e3
    tokens_per_s = B * args.steps / dt
    step_frac = mean_bytes / (dt / args.steps) / (HBM_PEAK_GBS * 1e9)

    if executor == "persistent":
        # Dominant kernel: the decode-step kernel itself, one launch per step: the events around the timed
        # iterations time exactly those launches (gaps between launches included).
        kernel_s, kernel_bytes, kernel_name = ev_s / args.steps, mean_bytes, step_kernel_name(B)
    else:
        # Dominant kernel: the fused INT4 gate/up (SwiGLU) projection, 2 x [11008, 4096] nibbles per
        # launch.  Timed with events on the stream it runs on, over every layer's weights in turn
        # (1.4 GB in total, so no launch finds its weights in a cache).
        stream = torch.cuda.Stream()
        d, f = cfg["hidden_size"], cfg["intermediate_size"]
        reps = 10
        with torch.cuda.stream(stream):
            for blk in weights.blocks:
                K.w4a16_gemm_swiglu(dec.h, blk.mlp_in[0].w, blk.mlp_in[1].w, dec.act)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            g = torch.cuda.CUDAGraph()
            stream.synchronize()
            with torch.cuda.graph(g, stream=stream):
                for blk in weights.blocks:
                    K.w4a16_gemm_swiglu(dec.h, blk.mlp_in[0].w, blk.mlp_in[1].w, dec.act)
            g.replay()
            e0.record(stream)
            for _ in range(reps):
                g.replay()
            e1.record(stream)
        torch.cuda.synchronize()
        launches = reps * len(weights.blocks)
        kernel_s = e0.elapsed_time(e1) * 1e-3 / launches
        kernel_bytes = 2 * (d * f // 2 + 2 * f) + B * d * 2 + B * f * 2
        kernel_name = ("gemv_lds_kernel<FmtW4, 8, true>" if B <= 4 else
                       "gemv_wide_kernel<FmtW4, 3, true>" if B <= 16 else "gemv_mfma_kernel<FmtW4, MT, 8, true>") + \
            " (INT4 gate/up + SwiGLU)"
    achieved = kernel_bytes / kernel_s / 1e9

    out = {
        "metric": "decode tokens/s at Llama2-7B INT4 bs=1/16 + % of HBM roofline",
        "value": tokens_per_s, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int4 weights, f16 activations, f32 accumulation", "data": "synthetic",
        "config": {"workload": f"Llama2-7B INT4 greedy decode, batch {B}, timed context {t_first}..{t_first + args.steps - 1} "
                               f"after the {prompt}-token prompt (untimed, "
                               f"{'in one pass' if in_passes else 'token by token'}), "
                               f"{'F143' if args.fp8_cache else 'fp16'} KV cache of {MAX_LEN}",
                   "batch": B, "kv_cache_len": MAX_LEN, "executor": executor},
        "step_algorithmic_bytes": float(mean_bytes), "step_roofline_frac": step_frac,
        "roofline": {"bound": "hbm", "kernel": kernel_name,
                     "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                     **traffic_fields(B), "bytes_per_launch": kernel_bytes, "avg_launch_us": kernel_s * 1e6},
    }
    default_run = B == 1 and not args.copy_calibration
    if default_run and not args.no_batch16:
        # the metric names batch 1 and batch 16: the same model, prompt, step counts and executor at batch 16,
        # reported beside the headline; `value` stays the batch-1 figure
        del dec
        torch.cuda.empty_cache()
        B16 = 16
        dec16 = decoder(B16)
        dt16, ev16, bytes16, _ = timed_decode(dec16, B16)
        out["batch16"] = {"value": B16 * args.steps / dt16, "unit": "tokens/s", "ms_per_step": dt16 / args.steps * 1e3,
                          "executor": executor, "timed_context": [t_first, t_first + args.steps - 1],
                          "step_algorithmic_bytes": bytes16,
                          "step_roofline_frac": bytes16 / (dt16 / args.steps) / (HBM_PEAK_GBS * 1e9)}
        if executor == "persistent":
            out["batch16"]["roofline"] = {"bound": "hbm", "kernel": step_kernel_name(B16),
                                          "achieved": bytes16 / (ev16 / args.steps) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                          "frac": bytes16 / (ev16 / args.steps) / 1e9 / HBM_PEAK_GBS, **traffic_fields(B16),
                                          "bytes_per_launch": bytes16, "avg_launch_us": ev16 / args.steps * 1e6}
        del dec16
    if args.copy_calibration:
        src = torch.empty(1 << 29, dtype=torch.float16, device="cuda").normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.neg(src, out=dst)
        torch.cuda.synchronize()
        del src, dst
    if default_run and not args.no_extras:
        # the other benchmark configurations, each bounded to a few seconds, under keys of their own
        dec = None
        del weights
        torch.cuda.empty_cache()

        def extra(key, fn):
            try:
                out[key] = fn()
            except Exception as e:          # the headline line is printed whatever happens here
                out[key] = {"error": f"{type(e).__name__}: {e}"}
                note(f"{key}: failed: {e}")
            torch.cuda.empty_cache()

        def single_operator():
            rows, ws = [], None
            for M in (1, 4, 16, 64):
                r, ws = gemm_measure(M, 192, 48, ws)
                rows.append(r)
                note(f"single operator M = {M}: {r['us_per_launch']:.2f} us")
            return {"workload": "X[M,4096] fp16 by W[4096,11008] packed INT4 with fp16 scales, 48 weight copies in turn",
                    "rows": rows}

        extra("single_operator", single_operator)
        extra("chatglm2_fp8_b8", lambda: brief(other_model_workload("chatglm2", 8, args.steps, args.warmup)))
        extra("rwkv_b1", lambda: brief(other_model_workload("rwkv", 1, args.steps, args.warmup)))
        extra("rwkv_b32", lambda: brief(other_model_workload("rwkv", 32, args.steps, args.warmup)))
        extra("gpt2_small", lambda: gpt2_small_workload(cpu=not args.no_cpu_baseline))
    if not args.no_cpu_baseline:
        note("CPU baseline: the numpy oracle of the headline graph on the host cores")
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))


if __name__ == "__main__":
    main()

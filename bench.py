#!/usr/bin/env python3
"""Benchmark of the speculative-decoding verify cycle on one MI355X.

A step is one pass of the hot path over one batch of BASELINE config 2: lossy entropy-gated tree
verification of 32 independent 64-node trees (bf16 logits [32, 64, 152064], threshold 0.3,
window 6) followed by top-k draft expansion (k = 16) over a same-shaped bf16 probability tensor
([2048, 1, 152064]).  Inputs are resident in HBM before the timed region.  Prints ONE JSON line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "verify_cycle_config2_hbm_counters.md")


def measured_traffic(kernel, batch, vocab):
    """HBM bytes per launch of `kernel` at the default workload, read from the committed counter summary (the rows
    of its first table: FETCH_SIZE and WRITE_SIZE in KiB per dispatch from two `rocprofv3 --pmc` runs; FETCH_SIZE
    counts the 16-byte-per-lane requests of these kernels at half their bytes, the calibration rows of the same
    table show it, hence the factor 2).  None for any other size, or when the summary does not name the kernel: the
    figure is a property of the profiled build, not of this run."""
    import re
    if (batch, vocab) != (32, 152064) or not os.path.exists(TRAFFIC_PROFILE):
        return None
    with open(TRAFFIC_PROFILE) as f:
        for line in f:
            m = re.match(r"\|\s*`subspec::" + re.escape(kernel) + r"[^|]*\|\s*([\d,\.]+)\s*\|\s*([\d,\.]+)\s*\|", line)
            if m:
                fetch_kib, write_kib = (float(g.replace(",", "")) for g in m.groups())
                return int(fetch_kib * 1024 * 2.0 + write_kib * 1024)
    return None


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--batch", type=int, default=32, help="trees per step (config 2: 32)")
    ap.add_argument("--vocab", type=int, default=152064)
    ap.add_argument("--cpu-trees", type=int, default=4, help="trees in the bounded CPU-baseline sample")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="lower bound of CPU-baseline work")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-e2e", action="store_true", help="default workload: leave out the bounded config-5 end-to-end block")
    ap.add_argument("--e2e-tokens", type=int, default=256,
                    help="default workload: new tokens of the config-5 runs of the e2e block that stream layers 14-27 with random "
                         "weights (256 is what BASELINE config 5 names: about 30 s per run)")
    ap.add_argument("--e2e-tokens-other", type=int, default=32,
                    help="default workload: new tokens of the other runs of the e2e block (all layers resident; agreeing draft)")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="also run three plain copies of the logits tensor (known size) so that hardware byte counters "
                         "collected by rocprofv3 --pmc can be scaled")
    ap.add_argument("--new-tokens", type=int, default=256, help="e2e workload: tokens to generate")
    ap.add_argument("--checkpoint", default=None,
                    help="e2e workload: local HuggingFace checkpoint directory (config.json + *.safetensors, Qwen2 / "
                         "Llama naming) to use instead of random-init weights of the Qwen2.5-7B shape")
    ap.add_argument("--agreeing-draft", action="store_true",
                    help="e2e workload: give the target the draft's dequantized int4 weights, so that draft and target agree "
                         "except for rounding: the high-acceptance end of the cycle (random weights alone accept about one "
                         "token per cycle)")
    ap.add_argument("--generator", default="v1", choices=["v1", "v2"],
                    help="e2e workload: v1 = speculate / verify cycle; v2 = the draft keeps extending the tree while the "
                         "target waits for streamed layers (post-speculation)")
    ap.add_argument("--postspec-steps", type=int, default=None,
                    help="e2e workload, generator v2: force this many post-speculation steps per target forward "
                         "(default: as many as fit into the waits for streamed layers)")
    ap.add_argument("--tree-depth", type=int, default=None, help="e2e workload: draft tree depth (default 8; 7 for generator v2)")
    ap.add_argument("--tree-k", type=int, default=8, help="e2e workload: children kept per level")
    ap.add_argument("--max-verify-tokens", type=int, default=64,
                    help="e2e workload: cap on the nodes verified per cycle (0: the whole tree); the reference's offloading "
                         "configurations use depth 48, k 6 and no cap: --tree-depth 48 --tree-k 6 --max-verify-tokens 0")
    ap.add_argument("--hqq-optimize", action="store_true",
                    help="e2e workload: refine the draft's zero points with hqq's proximal solver (what the reference's "
                         "quantizer does by default; worth it for real weights, --checkpoint)")
    ap.add_argument("--draft-graph", action="store_true",
                    help="e2e workload: replay each speculation (all draft levels) from a captured HIP graph")
    ap.add_argument("--keep-layers", type=int, default=14, help="e2e workload: target layers kept resident; the rest stream")
    ap.add_argument("--ring-slabs", type=int, default=4,
                    help="e2e workload: device slabs of the streaming ring (layers the copies may run ahead of compute)")
    ap.add_argument("--workload", default="verify-cycle", choices=["verify-cycle", "attention", "int4", "dense", "greedy", "sampling", "topk", "e2e", "tree-forward"],
                    help="verify-cycle (default, BASELINE config 2) is the benchmark line; the others time one "
                         "kernel family of configs 1, 3 and 4 and print one JSON line per shape")
    return ap.parse_args()


def _time_us(fn, steps, warmup):
    """(entry-point latency, dominant-kernel duration) of fn() in microseconds; events on the launch
    stream, the kernel duration from the library's event pair around its dominant kernel."""
    import torch
    from subspec_amd import _lib as L
    lib = L.lib()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    call_us = 1e3 * e0.elapsed_time(e1) / steps
    lib.subspec_profile_enable(1)
    for _ in range(min(steps, 64)):
        fn()
    torch.cuda.synchronize()
    lib.subspec_profile_enable(0)
    kern = sorted(lib.subspec_profile_read_ms(i) for i in range(lib.subspec_profile_count()))
    kernel_us = 1e3 * kern[len(kern) // 2] if kern else call_us
    return call_us, kernel_us


def _kernel_line(name, workload, call_us, kernel_us, nbytes, flops, kernel, bound="hbm", extra=None, dtype="bf16"):
    """One JSON line for a kernel family; `roofline` prices the dominant kernel against the bound named."""
    gbs = nbytes / (kernel_us * 1e-6) / 1e9
    tfl = flops / (kernel_us * 1e-6) / 1e12
    if bound == "hbm":
        roof = {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None}
    else:
        roof = {"bound": "mfma", "achieved": round(tfl, 1), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": round(tfl / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None}
    roof.update(kernel=kernel, kernel_us=round(kernel_us, 2), bytes_per_launch=nbytes, flops_per_launch=flops,
                hbm_frac=round(gbs / HBM_PEAK_GBS, 4), mfma_frac=round(tfl / MFMA_BF16_PEAK_TFLOPS, 4))
    line = {"metric": name, "value": round(call_us, 2), "unit": "us", "n_gpus": 1, "higher_is_better": False,
            "data": "synthetic", "dtype": dtype, "config": dict({"workload": workload}, **(extra or {})),
            "roofline": roof}
    print(json.dumps(line), flush=True)


def _rotating(make_call, n_copies):
    """fn() that uses copy 0, 1, 2, ... of the weights in turn: with enough copies (more bytes than the 256 MB
    memory-side cache plus the L2s hold) every call streams its weights from HBM, as inside a model where the
    other layers' weights pass through the caches between two uses of the same matrix."""
    state = [0]

    def fn():
        make_call(state[0] % n_copies)
        state[0] += 1
    return fn


COLD_BYTES = 640 << 20


def bench_attention(args):
    import torch
    from subspec_amd import ops, workloads as W
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(0)
    parents, _, _ = W.random_tree(g, n=64, max_depth=8, max_children=4, vocab=1000, chain_depth=8)
    anc = ops.ancestor_bits_tensor(parents, device=dev)
    for B in (1, 8):
        q = torch.randn(B, 28, 64, 128, device=dev).to(torch.bfloat16)
        # a different layer's cache on every call (rotation over > 640 MB), as in a forward through 28 layers
        copies = max(2, COLD_BYTES // (2 * B * 4 * 4160 * 128 * 2) + 1)
        ks = [torch.randn(B, 4, 4160, 128, device=dev).to(torch.bfloat16) for _ in range(copies)]
        vs = [torch.randn(B, 4, 4160, 128, device=dev).to(torch.bfloat16) for _ in range(copies)]
        need = ops.L.lib().subspec_tree_attention_workspace(B, 28, 4, 64, 4096, 64)
        ws = torch.empty(max(need, 256), dtype=torch.uint8, device=dev)
        call_us, kernel_us = _time_us(_rotating(lambda i: ops.tree_attention(q, ks[i], vs[i], anc, 4096, workspace=ws), copies),
                                      max(args.steps, copies), args.warmup)
        nbytes = B * (2 * 4 * 4160 * 128 * 2 + 2 * 28 * 64 * 128 * 2)
        # 3.82 GFLOP per sequence over 9.44 MB: at 405 FLOP/B the shape sits above the ridge (310 FLOP/B)
        _kernel_line("tree-masked GQA attention latency",
                     f"BASELINE config 3, B={B}: q [B,28,64,128], KV [B,4,4160,128] bf16, another cache every call ({copies} copies)",
                     call_us, kernel_us, nbytes, B * 4 * 64 * 28 * 4160 * 128,
                     "subspec::tree_attention_pp_kernel" if B > 1 else "subspec::tree_attention32_kernel", bound="mfma",
                     extra={"batch": B})
        del ks, vs
    # the same sequence out of a paged pool (16-token pages in shuffled order)
    page_len, n_pages, max_pages = 16, 4160 // 16, 300
    layer = torch.randn(max_pages, 2, page_len, 4, 128, device=dev).to(torch.bfloat16)
    pages = torch.randperm(max_pages, device=dev)[:n_pages].to(torch.int32)
    q = torch.randn(1, 28, 64, 128, device=dev).to(torch.bfloat16)
    need = ops.L.lib().subspec_tree_attention_workspace(1, 28, 4, 64, 4096, 64)
    ws = torch.empty(max(need, 256), dtype=torch.uint8, device=dev)
    call_us, kernel_us = _time_us(lambda: ops.tree_attention_paged(q, layer, pages, anc, 4096, workspace=ws), args.steps, args.warmup)
    _kernel_line("tree-masked GQA attention latency, paged KV", "config 3 shape, B=1, KV pool [300,2,16,4,128] bf16, shuffled pages",
                 call_us, kernel_us, 2 * 4 * 4160 * 128 * 2 + 2 * 28 * 64 * 128 * 2, 4 * 64 * 28 * 4160 * 128,
                 "subspec::tree_attention32_kernel", bound="mfma", extra={"batch": 1, "page_len": page_len})


def bench_int4(args):
    import torch
    from subspec_amd import ops, quant
    dev = torch.device("cuda:0")
    for N, K in ((4608, 3584), (3584, 3584), (37888, 3584), (3584, 18944)):
        W_ = torch.randn(N, K, device=dev) * 0.02
        wq, sz = quant.pack_tiled(*quant.quantize_int4_g64(W_))
        del W_
        copies = max(2, COLD_BYTES // (wq.numel() * 4) + 1)
        wqs, szs = [wq.clone() for _ in range(copies)], [sz.clone() for _ in range(copies)]
        for M in (1, 8, 16, 64):                          # 8: one draft level at top-k 8
            x = torch.randn(M, K, device=dev).to(torch.bfloat16)
            ws = torch.empty(max(ops.L.lib().subspec_int4_linear_workspace(M, N, K), 256), dtype=torch.uint8, device=dev)
            warm_us, warm_kernel_us = _time_us(lambda: ops.int4_linear(x, wq, sz, N, workspace=ws), args.steps, args.warmup)
            call_us, kernel_us = _time_us(_rotating(lambda i: ops.int4_linear(x, wqs[i], szs[i], N, workspace=ws), copies),
                                          max(args.steps, copies), args.warmup)
            nbytes = N * K // 2 + N * (K // 64) * 4 + M * (K + N) * 2
            _kernel_line("int4 g64 linear latency", f"BASELINE config 4: {K}->{N}, M={M}, bf16 activations, weights streamed "
                         f"from HBM (rotating over {copies} copies)", call_us, kernel_us, nbytes, 2 * M * N * K,
                         "subspec::int4_rows8_long_kernel" if (M <= 8 and K > 3584 and N >= 2048) else
                         "subspec::int4_rows8_kernel" if (M <= 16 and K > 2048) else
                         "subspec::int4_gemv_kernel" if M == 1 else "subspec::int4_gemm_kernel",
                         extra={"N": N, "K": K, "M": M, "same_weights_every_call_us": round(warm_us, 2),
                                "same_weights_every_call_kernel_us": round(warm_kernel_us, 2)})
        del wqs, szs


def bench_dense(args):
    """The target model's projections in the tree-decoding forward (bf16; 8 and 64 rows, and the 289 rows of a depth-48,
    k-6 tree), next to the library GEMM (torch F.linear) on the same operands; weights streamed from HBM as in
    bench_int4."""
    import torch
    import torch.nn.functional as F
    from subspec_amd import ops
    dev = torch.device("cuda:0")
    for N, K in ((4608, 3584), (3584, 3584), (37888, 3584), (3584, 18944)):
        copies = max(2, COLD_BYTES // (N * K * 2) + 1)
        wl = [(torch.randn(N, K, device=dev) * 0.02).to(torch.bfloat16) for _ in range(copies)]
        for M in (8, 64, 289):
            x = torch.randn(M, K, device=dev).to(torch.bfloat16)
            steps = max(args.steps, copies)
            call_us, kernel_us = _time_us(_rotating(lambda i: ops.dense_linear(x, wl[i]), copies), steps, args.warmup)
            lib_us, _ = _time_us(_rotating(lambda i: F.linear(x, wl[i]), copies), steps, args.warmup)
            _kernel_line("dense 16-bit linear latency", f"target layer projection {K}->{N}, M={M}, bf16, weights streamed from "
                         f"HBM (rotating over {copies} copies)", call_us, kernel_us, N * K * 2 + M * (K + N) * 2, 2 * M * N * K,
                         "subspec::dense_gemm_kernel" if M <= 32 else "subspec::dense_wide_kernel",
                         extra={"N": N, "K": K, "M": M, "library_gemm_call_us": round(lib_us, 2)})
        del wl


def e2e_runs(args, runs, new_tokens, say=lambda *_: None):
    """BASELINE config 5: random-init Qwen2.5-7B-shaped decoder, target bf16 with layers 14-27 streamed from pinned host
    memory every forward, substitute draft int4 g64 resident, depth-8 / k-8 tree capped at 64 nodes, prompt 2048 random
    ids; exact and lossy verification.  `runs`: (keep_layers, agreeing_draft) pairs, each generated with both
    verification methods; a run may carry its own token count as a third element.  Returns one JSON-ready line per generation."""
    import torch
    from subspec_amd.cache import create_kv_cache
    from subspec_amd.draft import SubSpecSDDraftModel
    from subspec_amd.generator import SubSpecSDGenerator
    from subspec_amd.generator_v2 import SubSpecSDGeneratorV2
    from subspec_amd import quant
    from subspec_amd.model import QUANTIZED, DecoderConfig, build_models, init_weights, load_hf_checkpoint
    from subspec_amd.utils import DraftParams
    from subspec_amd.wandb_logger import wandb_logger
    dev = "cuda:0"
    lines = []
    base = None
    default_tokens = new_tokens
    for run in runs:
        keep_layers, agreeing = run[0], run[1]
        new_tokens = run[2] if len(run) > 2 else default_tokens
        tree = run[3] if len(run) > 3 else None             # (depth, k, node cap or None) of this run's draft tree
        t0 = time.perf_counter()
        if args.checkpoint:
            cfg, weights = load_hf_checkpoint(args.checkpoint, device=dev)
        else:
            cfg = DecoderConfig()
            if base is None:
                base = init_weights(cfg, 0, dev)
            weights = {**base, "layers": [dict(w) for w in base["layers"]]}
        if agreeing:
            for w in weights["layers"]:
                for name in QUANTIZED:
                    t = w[name + ".weight"]
                    w[name + ".weight"] = quant.dequantize(*quant.quantize_int4_g64(t)).to(t.dtype)
        kv = create_kv_cache("static", max_cache_len=2048 + new_tokens + 512 + 8, config=cfg, device=dev, dtype=torch.bfloat16)
        target, draft, _ = build_models(cfg, kv, seed=0, device=dev, first_streamed=min(keep_layers, cfg.num_hidden_layers),
                                        weights=weights, hqq_optimize=args.hqq_optimize,
                                        n_slabs=getattr(args, "ring_slabs", 4))
        say(f"# models built in {time.perf_counter() - t0:.1f} s (resident target layers: {keep_layers}, agreeing draft: {agreeing})")
        prompt = torch.randint(0, cfg.vocab_size, (1, 2048), generator=torch.Generator().manual_seed(0)).to(dev)
        warm = False
        for method, vk in (("exact", None), ("lossy", dict(threshold=0.3, window_size=6, threshold_method="entropy"))):
            v2 = args.generator == "v2"
            depth = args.tree_depth or (7 if v2 else 8)
            cap = args.max_verify_tokens or None
            tree_k = args.tree_k
            if tree is not None:
                depth, tree_k, cap = tree
            gen = (SubSpecSDGeneratorV2 if v2 else SubSpecSDGenerator)(
                target, None, SubSpecSDDraftModel(draft),
                DraftParams(temperature=0.2, max_depth=depth, topk_len=tree_k, max_verify_tokens=cap),
                generator_kwargs=dict(verify_method=method, verify_kwargs=vk, draft_graph=bool(getattr(args, "draft_graph", False)),
                                      **(dict(postspec_steps=args.postspec_steps) if v2 else {})))
            if not warm:
                # one untimed prefill (a generation of one token): the first pass through the GEMM library in a new
                # process selects and loads its kernels (290 ms against 42 ms for every later prefill of this prompt),
                # which is no property of the cycle
                kv.reset()
                gen.generate(prompt, max_new_tokens=1, do_sample=False, past_key_values=kv)
                torch.cuda.synchronize()
                warm = True
            kv.reset()
            wandb_logger.clear_log_data()
            if target.streamer is not None:
                target.streamer.bytes_streamed = 0
            gen.generate(prompt, max_new_tokens=new_tokens, do_sample=False, past_key_values=kv)
            log = dict(wandb_logger.log_data)
            cycle_s = log.get("avg_draft_time", 0) + log.get("avg_target_time", 0) + log.get("avg_verify_time", 0)
            h2d = target.streamer.bytes_streamed if target.streamer else 0
            lines.append({
                "metric": "accepted tokens/sec, end-to-end speculative cycle", "value": round(log["tput"], 2),
                "unit": "tokens/s", "n_gpus": 1, "higher_is_better": True, "dtype": "bf16",
                "data": ("synthetic prompt, weights from " + args.checkpoint if args.checkpoint else "synthetic")
                        + (", target = the draft's dequantized int4 weights" if agreeing else ""),
                "config": {"workload": f"BASELINE config 5: {'checkpoint' if args.checkpoint else 'Qwen2.5-7B shape'}, "
                                       + ("all layers resident" if keep_layers >= cfg.num_hidden_layers else
                                          f"layers {keep_layers}-{cfg.num_hidden_layers - 1} streamed")
                                       + f", int4 draft, depth {depth}, k {tree_k}, "
                                       + (f"<={cap} nodes" if cap else f"{1 + depth * tree_k} nodes") + f", prompt 2048, {new_tokens} new tokens, verify {method}"
                                       + (", post-speculating driver" if v2 else ""),
                           "verify_method": method, "generator": args.generator,
                           "tree": f"depth {depth}, k {tree_k}, " + (f"<={cap} nodes" if cap else f"{1 + depth * tree_k} nodes"),
                           "draft_graph_replays": gen.draft_model.graph_replays, "resident_target_layers": min(keep_layers, cfg.num_hidden_layers),
                           "ring_slabs": (target.streamer.n_slabs if target.streamer is not None else 0),
                           "agreeing_draft": bool(agreeing),
                           **({"post_verify_count": log["post_verify_count"], "speculate_count": log["speculate_count"]} if v2 else {}), "n_iter": log["n_iter"], "n_tokens": log["n_tokens"],
                           "tokens_per_cycle": round(log["avg_sampled"], 3),
                           "avg_draft_s": round(log.get("avg_draft_time", 0), 5),
                           "avg_target_s": round(log.get("avg_target_time", 0), 5),
                           "avg_verify_s": round(log.get("avg_verify_time", 0), 6),
                           # tokens per second of the cycles alone (the prefill of the 2048-token prompt, which `value`
                           # includes as the reference's tput does, weighs heavily on a short generation)
                           "cycle_tokens_per_s": round(log["avg_sampled"] / cycle_s, 2) if cycle_s > 0 else None,
                           "elapsed_s": round(log["elapsed_time"], 3),
                           "host_to_device_GB": round(h2d / 1e9, 2),
                           "host_to_device_GB_per_s": round(h2d / 1e9 / log["elapsed_time"], 1) if h2d else 0.0}})
        del target, draft, kv, weights
        torch.cuda.empty_cache()
    return lines


def bench_tree_forward(args):
    """One target forward over the rows of a whole draft tree, all 28 layers resident, prefix 2048: 64 rows (the default
    verification window), 128, and the 289 rows of the reference's depth-48, k-6 tree
    (configs/exp_offloading/subspec_sd_qwen_7b.yaml:16-19) -- through the one-call dense layers, and module by module on
    library GEMMs with the same attention kernel."""
    import torch
    from subspec_amd import ops, workloads as W
    from subspec_amd.cache import create_kv_cache
    from subspec_amd.model import DecoderConfig, build_models
    dev = "cuda:0"
    cfg = DecoderConfig()
    kv = create_kv_cache("static", max_cache_len=2048 + 400, config=cfg, device=dev, dtype=torch.bfloat16)
    target, _, _ = build_models(cfg, kv, seed=0, device=dev, first_streamed=cfg.num_hidden_layers)
    g = torch.Generator().manual_seed(0)
    target.prefill(torch.randint(0, cfg.vocab_size, (2048,), generator=g).to(dev), 0)
    weight_bytes = sum(t.numel() * 2 for w in target.layers for n_, t in w.items() if n_.endswith("_proj.weight"))
    for n in (64, 128, 289):
        parents, _, depths = W.random_tree(g, n=n, max_depth=48, max_children=6, vocab=cfg.vocab_size, chain_depth=8)
        toks = torch.randint(0, cfg.vocab_size, (n,), generator=g).to(dev)
        anc = ops.ancestor_bits_tensor(parents, device=dev)
        d = torch.tensor(depths, device=dev)
        times = {}
        for native in (True, False):
            target.use_native_layers = native
            times[native], _ = _time_us(lambda: target.tree_forward(toks, d, anc, 2048), max(5, args.steps // 2), 2)
        target.use_native_layers = True
        flops = 2 * n * weight_bytes // 2
        print(json.dumps({"metric": "target forward over the rows of a draft tree", "value": round(times[True] / 1e3, 3), "unit": "ms",
                          "n_gpus": 1, "higher_is_better": False, "data": "synthetic", "dtype": "bf16",
                          "config": {"workload": f"Qwen2.5-7B shape, 28 resident layers, prefix 2048, {n} tree rows, one-call dense layers",
                                     "rows": n, "module_by_module_library_gemm_ms": round(times[False] / 1e3, 3),
                                     "layer_weight_GB": round(weight_bytes / 1e9, 2),
                                     "weights_over_time_TB_per_s": round(weight_bytes / (times[True] * 1e-6) / 1e12, 2),
                                     "projection_TFLOP_per_s": round(flops / (times[True] * 1e-6) / 1e12, 1)}}), flush=True)


def bench_e2e(args):
    for line in e2e_runs(args, [(args.keep_layers, args.agreeing_draft)], args.new_tokens,
                         say=lambda m: print(m, file=sys.stderr, flush=True)):
        print(json.dumps(line), flush=True)


def e2e_block(args):
    """The bounded config-5 runs the default line carries: `--e2e-tokens` new tokens after the 2048-token prompt, layers
    14-27 streamed (the configuration BASELINE names) and all layers resident, random weights, exact and lossy; plus
    the streamed cycle with a draft that agrees with its target (the high-acceptance end random weights cannot show)."""
    keys = ("verify_method", "resident_target_layers", "agreeing_draft", "tree", "n_iter", "n_tokens", "tokens_per_cycle", "avg_draft_s",
            "avg_target_s", "avg_verify_s", "cycle_tokens_per_s", "elapsed_s", "host_to_device_GB", "host_to_device_GB_per_s")
    out = {"workload": f"BASELINE config 5, Qwen2.5-7B shape (28 layers, hidden 3584, 28/4 heads, FFN 18944, vocab 152064), int4 g64 "
                       f"draft, depth 8, k 8, <=64 nodes, prompt 2048, {args.e2e_tokens} new tokens with layers 14-27 streamed and random "
                       f"weights, {args.e2e_tokens_other} in the other runs (the last of them with the depth-48, k-6, 289-node tree); "
                       "tokens_per_s = new tokens / "
                       "whole generate() including the prefill, cycle_tokens_per_s = tokens per cycle / (draft + target + verify)",
           "runs": []}
    # the last run: the tree of the reference's offloading configuration (depth 48, k 6, all 289 nodes verified in one
    # target forward; configs/exp_offloading/subspec_sd_qwen_7b.yaml:16-19), all layers resident
    for line in e2e_runs(args, [(14, False, args.e2e_tokens), (28, False, args.e2e_tokens_other), (14, True, args.e2e_tokens_other),
                                (28, False, args.e2e_tokens_other, (48, 6, None))],
                         args.e2e_tokens):
        out["runs"].append(dict({"tokens_per_s": line["value"]}, **{k: line["config"][k] for k in keys}))
    return out


def bench_topk(args):
    """Top-16 expansion of 2048 x 152064 bf16 rows on three kinds of rows: the default workload's (softmax of scaled
    Gaussians), near-uniform rows (every probability within 0.1 % of 1 / V: in bf16 almost all entries of a row are
    EQUAL, the ballot threshold of the slice kernel rejects nothing and its prune steps do the work), and one-hot
    rows.  The second is the worst case for the screening."""
    import torch
    from subspec_amd import ops
    dev = torch.device("cuda:0")
    rows, V, k = 2048, 152064, 16
    g = torch.Generator(device=dev).manual_seed(5)
    kinds = {}
    z = torch.randn(rows, 1, V, generator=g, device=dev) * (torch.rand(rows, 1, 1, generator=g, device=dev) * 2.5 + 0.5)
    kinds["softmax of scaled Gaussians (the default workload's rows)"] = torch.softmax(z.to(torch.bfloat16), -1)
    del z
    kinds["near-uniform rows (1 / V within 0.1 %)"] = ((1.0 + 1e-3 * torch.rand(rows, 1, V, generator=g, device=dev)) / V).to(torch.bfloat16)
    hot = torch.zeros(rows, 1, V, device=dev, dtype=torch.bfloat16)
    hot[torch.arange(rows, device=dev), 0, torch.randint(0, V, (rows,), generator=g, device=dev)] = 1
    kinds["one-hot rows"] = hot
    parent = torch.rand(rows, 1, generator=g, device=dev).to(torch.bfloat16)
    ws = torch.empty(ops.L.lib().subspec_topk_expand_workspace(rows, 1, V, k), dtype=torch.uint8, device=dev)
    for name, probs in kinds.items():
        call_us, kernel_us = _time_us(lambda: ops.topk_expand(probs, parent, k, workspace=ws), args.steps, args.warmup)
        _kernel_line("top-k expansion latency", f"top-16 of 2048 x 152064 bf16 rows, {name}", call_us, kernel_us, rows * V * 2, 0,
                     "subspec::topk_slice_kernel", extra={"rows": name})


def bench_greedy(args):
    import torch
    from subspec_amd import ops, workloads as W
    dev = torch.device("cuda:0")
    cfg = W.greedy_config(0, device=dev)
    tok = torch.tensor(cfg["tokens"], dtype=torch.int32, device=dev)
    par = torch.tensor(cfg["parents"], dtype=torch.int32, device=dev)
    ws = torch.empty(ops.L.lib().subspec_tree_verify_workspace(1, 64, 152064, 0), dtype=torch.uint8, device=dev)
    fresh_us, _ = _time_us(lambda: ops.tree_verify(cfg["logits"], tok, par, workspace=ws), args.steps, args.warmup)
    # a decoding loop hands the same output tensors back in: the call then allocates nothing
    out = ops.tree_verify(cfg["logits"], tok, par, workspace=ws)
    call_us, kernel_us = _time_us(lambda: ops.tree_verify(cfg["logits"], tok, par, workspace=ws, out=out), args.steps, args.warmup)
    # ... and a prepared call has its checks and argument conversions behind it as well
    prepared = ops.PreparedTreeVerify(cfg["logits"], tok, par, workspace=ws, out=out)
    prepared_us, _ = _time_us(prepared.call, args.steps, args.warmup)
    _kernel_line("greedy tree verify latency", "BASELINE config 1: fp32 logits [64,152064], 64-node tree", prepared_us,
                 kernel_us, 64 * 152064 * 4, 0, "subspec::row_partial_kernel",
                 extra={"call": "ops.PreparedTreeVerify (launches only)", "call_us_tree_verify_reused_outputs": round(call_us, 2),
                        "call_us_tree_verify_fresh_outputs": round(fresh_us, 2)}, dtype="f32")


def bench_sampling(args):
    """Config 2's logits verified against a SAMPLED target (temperature 0.8): statistics pass + one
    Philox draw per row + walk.  The draw re-reads the rows, so its algorithmic bytes are the rows again."""
    import torch
    from subspec_amd import ops, workloads as W
    dev = torch.device("cuda:0")
    cfg = W.lossy_config(0, batch=32, device=dev)
    tok = torch.tensor(cfg["tokens"], dtype=torch.int32, device=dev)
    par = torch.tensor(cfg["parents"], dtype=torch.int32, device=dev)
    ws = torch.empty(ops.L.lib().subspec_tree_verify_workspace(32, 64, 152064, 2), dtype=torch.uint8, device=dev)
    step = [0]

    def fn():
        step[0] += 1
        ops.tree_verify(cfg["logits"], tok, par, workspace=ws, verify_method="exact", do_sample=True, temperature=0.8,
                        seed=1, offset=step[0])

    call_us, kernel_us = _time_us(fn, args.steps, args.warmup)
    _kernel_line("sampling tree verify latency", "config 2 logits [32,64,152064] bf16, sampled target (T = 0.8), exact walk",
                 call_us, kernel_us, 32 * 64 * 152064 * 2, 0, "subspec::row_sample_kernel")


def cpu_baseline(cfg, probs_rows, parent_rows, n_trees, min_seconds):
    """The oracle (torch-on-CPU restatement of the reference path) on a bounded sample of the same
    workload: `n_trees` trees of the batch + their 64 top-k rows each, repeated until at least
    `min_seconds` of CPU work has been timed."""
    import torch
    from oracle import topk as ot
    from oracle import verify as ov

    # threads: the CPUs this process may run on, capped by the thread limit the host sets for its jobs (OMP_NUM_THREADS)
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    if os.environ.get("OMP_NUM_THREADS", "").isdigit():
        cores = max(1, min(cores, int(os.environ["OMP_NUM_THREADS"])))
    torch.set_num_threads(cores)
    cpu_model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            cpu_model = next((l.split(":", 1)[1].strip() for l in f if l.startswith("model name")), "unknown")
    except OSError:
        pass
    vk = dict(threshold=cfg["threshold"], window_size=cfg["window_size"], threshold_method="entropy")
    logits = [cfg["logits"][b].cpu() for b in range(n_trees)]
    rows = probs_rows[: n_trees * 64].cpu()
    par = parent_rows[: n_trees * 64].cpu()

    def one_pass():
        toks = 0
        for b in range(n_trees):
            t, _, _ = ov.verify_logits(logits[b], cfg["tokens"][b], cfg["parents"][b], verify_method="lossy",
                                       verify_kwargs=vk)
            toks += len(t)
        ot.topk_expand_torch(rows, par, 16)
        return toks

    one_pass()                                         # warm-up
    t0 = time.perf_counter()
    passes = toks = 0
    while True:
        toks += one_pass()
        passes += 1
        el = time.perf_counter() - t0
        if el >= min_seconds:
            break
    return {
        "value": toks / el, "unit": "tokens/s", "cores": cores, "kind": "port", "cpu_model": cpu_model,
        "host_logical_cpus": os.cpu_count(),
        "sample": f"{n_trees} of the batch's trees (64 rows x 152064 each: softmax, argmax, entr, DP) + "
                  f"top-16 of their {n_trees * 64} rows, {passes} passes in {el:.1f} s",
        "ms_per_tree": 1e3 * el / (passes * n_trees),
    }


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build measures ONE GPU; --gpus must be 1 "
              "(each tree / sequence is independent, so N GPUs would each run this same kernel on 1/N of the batch)",
              file=sys.stderr)
        sys.exit(2)
    import torch
    from subspec_amd import _lib as L
    from subspec_amd import ops, workloads as W

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    L.lib()                                            # fail loudly when the HIP library is missing
    if args.workload != "verify-cycle":
        {"attention": bench_attention, "int4": bench_int4, "dense": bench_dense, "greedy": bench_greedy, "sampling": bench_sampling, "topk": bench_topk,
         "e2e": bench_e2e, "tree-forward": bench_tree_forward}[args.workload](args)
        return
    dev = torch.device("cuda:0")
    B, V, n, k = args.batch, args.vocab, 64, 16

    cfg = W.lossy_config(seed=0, batch=B, vocab=V, device=dev)
    tok = torch.tensor(cfg["tokens"], dtype=torch.int32, device=dev)
    par = torch.tensor(cfg["parents"], dtype=torch.int32, device=dev)
    g = torch.Generator(device=dev).manual_seed(77)
    draft = torch.empty(B * n, 1, V, dtype=torch.bfloat16, device=dev)
    for b in range(B):                                 # draft probabilities: softmax of scaled Gaussians
        z = torch.randn(n, 1, V, generator=g, device=dev) * (torch.rand(n, 1, 1, generator=g, device=dev) * 2.5 + 0.5)
        draft[b * n:(b + 1) * n] = torch.softmax(z.to(torch.bfloat16), -1)
        del z
    parent_probs = torch.rand(B * n, 1, generator=g, device=dev).to(torch.bfloat16)
    lib = L.lib()
    ws_v = torch.empty(lib.subspec_tree_verify_workspace(B, n, V, L.BF16), dtype=torch.uint8, device=dev)
    ws_t = torch.empty(lib.subspec_topk_expand_workspace(B * n, 1, V, k), dtype=torch.uint8, device=dev)

    def step():
        out = ops.tree_verify(cfg["logits"], tok, par, verify_method="lossy", threshold_method="entropy",
                              threshold=cfg["threshold"], window_size=cfg["window_size"], workspace=ws_v)
        top = ops.topk_expand(draft, parent_probs, k, workspace=ws_t)
        return out, top

    for _ in range(args.warmup):
        out, top = step()
    torch.cuda.synchronize()
    if args.pmc_calibration:
        for _ in range(3):
            calib = cfg["logits"].clone()                # copy kernel: reads and writes B*n*V*2 bytes
        torch.cuda.synchronize()
        del calib

    # timed region: exactly `steps` steps, synchronised on both sides, nothing else on the stream
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        out, top = step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0

    # outside the timed region: the same steps with events around each call (an event record costs the stream about
    # 5 us, three of them per step would inflate the timed step by 6 %), on the stream the kernels are launched on
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(args.steps)]
    for i in range(args.steps):
        ev[i][0].record()
        ops.tree_verify(cfg["logits"], tok, par, verify_method="lossy", threshold_method="entropy",
                        threshold=cfg["threshold"], window_size=cfg["window_size"], workspace=ws_v)
        ev[i][1].record()
        ops.topk_expand(draft, parent_probs, k, workspace=ws_t)
        ev[i][2].record()
    torch.cuda.synchronize()

    # and once more with the library's event pair around the dominant kernel of every call
    lib.subspec_profile_enable(1)
    for i in range(args.steps):
        step()
    torch.cuda.synchronize()
    lib.subspec_profile_enable(0)
    n_prof = lib.subspec_profile_count()
    kern = [lib.subspec_profile_read_ms(i) for i in range(n_prof)]
    row_kernel_ms = sum(kern[0::2]) / max(1, len(kern[0::2]))     # calls alternate: verify, top-k
    topk_kernel_ms = sum(kern[1::2]) / max(1, len(kern[1::2]))

    verify_ms = sum(e[0].elapsed_time(e[1]) for e in ev) / args.steps
    topk_ms = sum(e[1].elapsed_time(e[2]) for e in ev) / args.steps
    counts = out["counts"].cpu()
    assert int(counts[:, 3].abs().sum()) == 0, "verifier reported a broken tree"
    tokens_per_step = int(counts[:, 0].sum())          # accepted draft tokens + one bonus token per tree
    accepted_per_step = int(counts[:, 1].sum())
    ms_per_step = 1e3 * elapsed / args.steps
    bytes_verify = B * n * V * 2
    bytes_topk = B * n * V * 2

    def roof(nbytes, ms, which):
        gbs = nbytes / (ms * 1e-3) / 1e9
        return {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": measured_traffic(which, B, V),
                "traffic_source": "profiles/verify_cycle_config2_hbm_counters.md (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of "
                                  "the profiled build, not re-measured in this run)"}

    result = {
        "metric": "accepted tokens/sec + verify-cycle latency (Qwen2.5-7B shape); % HBM roofline",
        "value": round(tokens_per_step / (ms_per_step * 1e-3), 1),
        "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "BASELINE config 2: lossy entropy-gated tree verify (theta 0.3, window 6) of "
                               f"{B} trees x 64 nodes x {V} bf16 logits + top-16 expansion of {B * n} x {V} bf16 rows",
                   "trees": B, "nodes": n, "vocab": V, "topk": k,
                   "tokens_per_step": tokens_per_step, "accepted_draft_tokens_per_step": accepted_per_step,
                   "verify_ms": round(verify_ms, 4), "topk_ms": round(topk_ms, 4)},
        "roofline": dict(roof(bytes_verify, row_kernel_ms, "row_partial_kernel"), kernel="subspec::row_partial_kernel",
                         bytes_per_launch=bytes_verify, kernel_ms=round(row_kernel_ms, 4),
                         sequence_frac=round(bytes_verify / (verify_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)),
        "roofline_topk": dict(roof(bytes_topk, topk_kernel_ms, "topk_slice_kernel"), kernel="subspec::topk_slice_kernel",
                              bytes_per_launch=bytes_topk, kernel_ms=round(topk_kernel_ms, 4),
                              sequence_frac=round(bytes_topk / (topk_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)),
    }
    cfg_cpu = None
    if not args.no_cpu_baseline:
        cfg_cpu = dict(cfg)
        result["cpu_baseline"] = cpu_baseline(cfg_cpu, draft, parent_probs, min(args.cpu_trees, B), args.cpu_seconds)
    if not args.no_e2e:
        cfg = cfg_cpu = draft = parent_probs = out = top = ws_v = ws_t = ev = None     # free the config-2 tensors
        torch.cuda.empty_cache()
        result["e2e_config5"] = e2e_block(args)
    print(json.dumps(result))


if __name__ == "__main__":
    main()

#!/usr/bin/env python3
"""Tree-verification step benchmark on one MI355X.

A step is one full verification forward of a random-init Qwen2.5-7B-shaped 4-bit (group 64)
target over 32 tree tokens (root + 31 nodes of a seeded random tree) against a 2048-token
fp16 KV prefix: embedding, 28 decoder layers, output head, per-node argmax, greedy
longest-accepted-path selection and KV compaction, replayed as one HIP graph with every
input resident in HBM.  Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--sweep]

--sweep additionally prints (to stderr) the per-shape QMM table for M in {1,8,16,24,32}.

  python bench.py --loop [--steps 300]

measures the end-to-end greedy tree loop instead (a second workload with a line of its own):
random-init Qwen2.5-0.5B-shaped drafter, Llama-3-8B-shaped target, 512-token random prompt,
depth 3, 31 draft nodes; every step (draft pass, expansion, tree layout, verification,
acceptance, KV compaction) is one HIP-graph replay with the loop state on the device.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# HBM bytes per QMM launch of this workload: FETCH_SIZE + WRITE_SIZE from two rocprofv3 --pmc
# runs of this script, scaled by a copy kernel of known size.  `--traffic-from` turns the two
# counter files into this tracked record; the benchmark line quotes it with its source.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "qmm_traffic.json")
# Bound on max |logits - oracle| / RMS after all 28 layers (every operator alone meets 2e-2;
# tests/test_gpu_fullsize.py follows the growth through the layers: 0.005 after one layer,
# 0.03-0.035 after 28, the same for both forms of the matmul and both weight-rounding modes
# of the oracle).
FULL_DEPTH_BOUND = 6e-2
PREFIX = 2048
NODES = 32
ACCEPT_CHAIN = 3        # draft tokens of the benchmark tree that the target accepts (see tree_verify)


def write_traffic_record(fetch_csv, write_csv):
    """Turn the counter files of
        rocprofv3 --pmc FETCH_SIZE --output-format csv -d <dir> -o fetch -- python3 bench.py --headline-only --no-cpu --steps 2 --warmup 1 --calibrate-copy
        rocprofv3 --pmc WRITE_SIZE --output-format csv -d <dir> -o write -- python3 bench.py --headline-only --no-cpu --steps 2 --warmup 1 --calibrate-copy
    into profiles/qmm_traffic.json: mean counter value over the quantised-matmul dispatches,
    scaled by what the same counter reads for the 1 GiB copy that --calibrate-copy runs first."""
    import csv
    import subprocess
    rec = {}
    for name, path in (("FETCH_SIZE", fetch_csv), ("WRITE_SIZE", write_csv)):
        q, cp = [], []
        with open(path) as f:
            for r in csv.DictReader(f):
                if r["Counter_Name"] != name:
                    continue
                kn = r["Kernel_Name"]
                if any(k in kn for k in ("qmm_w4g64", "qmm_slab_w4g64", "qmm_burst_w4g64", "qmm_rows_tiled")):
                    q.append(float(r["Counter_Value"]))
                if "copyBuffer" in kn or "elementwise" in kn:
                    cp.append(float(r["Counter_Value"]))
        kib_per_count = 1048576.0 / max(cp)
        rec[name] = {"mean_per_launch": sum(q) / len(q), "dispatches": len(q),
                     "copy_1GiB_reads": max(cp), "kib_per_count": kib_per_count,
                     "bytes_per_launch": sum(q) / len(q) * kib_per_count * 1024}
    rec["traffic_bytes_per_launch"] = round(rec["FETCH_SIZE"]["bytes_per_launch"] + rec["WRITE_SIZE"]["bytes_per_launch"])
    try:
        rec["commit"] = subprocess.run(["git", "-C", ROOT, "rev-parse", "--short", "HEAD"], capture_output=True,
                                       text=True).stdout.strip() or None
    except OSError:
        rec["commit"] = None
    rec["command"] = ("rocprofv3 --pmc FETCH_SIZE|WRITE_SIZE --output-format csv -- python3 bench.py "
                      "--headline-only --no-cpu --steps 2 --warmup 1 --calibrate-copy")
    os.makedirs(os.path.dirname(TRAFFIC_FILE), exist_ok=True)
    with open(TRAFFIC_FILE, "w") as f:
        json.dump(rec, f, indent=1)
        f.write("\n")
    print(json.dumps(rec))


def read_traffic_record():
    try:
        with open(TRAFFIC_FILE) as f:
            rec = json.load(f)
        return rec["traffic_bytes_per_launch"], {"file": "profiles/qmm_traffic.json", "commit": rec.get("commit")}
    except (OSError, KeyError, ValueError):
        return None, None


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def set_omp_threads(n):
    import ctypes
    ctypes.CDLL("libgomp.so.1").omp_set_num_threads(int(n))


def qmm_bytes(M, N, K, n_out=None):
    """Algorithmic bytes of one 4-bit group-64 QMM: packed weights + fp16 scale and bias per
    64 weights (0.5625 B per weight) + fp16 activations in and out (the SwiGLU form writes
    n_out = N / 2 columns)."""
    return 0.5625 * N * K + 2.0 * M * (K + (N if n_out is None else n_out))


def qmm_shapes(args):
    D, I, V = args.hidden_size, args.intermediate_size, args.vocab_size
    H, G, hd = args.num_attention_heads, args.num_key_value_heads, args.head_dim
    per_layer = [("q", H * hd, D), ("k", G * hd, D), ("v", G * hd, D), ("o", D, H * hd),
                 ("gate", I, D), ("up", I, D), ("down", D, I)]
    return per_layer, ("lm_head", V, D)


def pass_bytes(args, M, prefix):
    """Algorithmic bytes of one pass of M rows through a model behind `prefix` cached tokens:
    every quantised product once (qmm_bytes) and the K / V rows of every layer read once."""
    per_layer, head = qmm_shapes(args)
    L, G, hd = args.num_hidden_layers, args.num_key_value_heads, args.head_dim
    mats = L * sum(qmm_bytes(M, n, k) for _, n, k in per_layer) + qmm_bytes(M, head[1], head[2])
    return mats + 2.0 * L * G * (prefix + M) * hd * 2


def graph_time_ms(torch, fn, reps, warm=2):
    """Capture fn() once in a HIP graph and time `reps` replays with events on the
    replay stream; returns the list of per-replay milliseconds."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        fn()
    for _ in range(warm):
        g.replay()
    torch.cuda.synchronize()
    out = []
    for _ in range(reps):
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        g.replay()
        e1.record()
        torch.cuda.synchronize()
        out.append(e0.elapsed_time(e1))
    return out, g


def main():
    global NODES
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--seed", type=int, default=1234)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline / full-size parity leg")
    ap.add_argument("--headline-only", action="store_true",
                    help="skip the two extra workloads (tree loop, prompt-pass matmul) that the default run "
                         "appends to the line as `loop` and `prompt_gemm`")
    ap.add_argument("--traffic-from", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"),
                    help="no benchmark: turn two rocprofv3 counter files into profiles/qmm_traffic.json")
    ap.add_argument("--slabs", default=None,
                    help="force the slab form of the matmul: e.g. qkv=8,o=8,down=32 (K steps per slab; "
                         "'' = streaming kernel everywhere; default: the library's choice)")
    ap.add_argument("--draft-slabs", default=None,
                    help="--loop: the same for the drafter's passes")
    ap.add_argument("--no-draft-folded", action="store_true",
                    help="--loop: the drafter's passes with one launch per operator instead of the small-row "
                         "products with norm / residual / SwiGLU folded in")
    ap.add_argument("--sweep", action="store_true", help="also print the per-shape QMM table to stderr")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="before anything else run one 1 GiB device copy (a kernel of known traffic: "
                         "1 GiB read + 1 GiB written) so that profiler byte counters can be scaled")
    ap.add_argument("--loop", action="store_true",
                    help="measure the end-to-end tree loop (drafter + target) instead of the verify step")
    ap.add_argument("--gemm", action="store_true",
                    help="measure the many-row (prompt pass) form of the quantised matmul instead")
    ap.add_argument("--small-m", action="store_true",
                    help="one-row products of the 7B projection shapes: the vector-ALU kernel beside the "
                         "matrix kernel (one JSON line; the A/B behind the dispatch rule for M = 1)")
    ap.add_argument("--attention", action="store_true",
                    help="tree-position rope + tree-masked attention alone (28 / 4 heads of 128, 32 tree tokens) "
                         "over 1024- and 2048-token prefixes, one JSON line")
    ap.add_argument("--cpu-qmm", action="store_true",
                    help="time the CPU restatement of single quantised matmuls on the host cores (cfg1 and the "
                         "7B projection shapes; one JSON line); no GPU work")
    ap.add_argument("--tree-tokens", type=int, default=NODES,
                    help="tree tokens of the verification step (root included; the headline is quoted on 32, "
                         "the reference's default tree has 40)")
    ap.add_argument("--depth", type=int, default=3, help="--loop: levels of the draft tree")
    ap.add_argument("--draft-nodes", type=int, default=31,
                    help="--loop: draft nodes verified per step (the reference's default is 39 at depth 5)")
    ap.add_argument("--self-draft", action="store_true",
                    help="with --loop: the target drafts for itself (high acceptance; exercises the "
                         "accept path at full size)")
    opt = ap.parse_args()
    if opt.gpus != 1:
        print("bench.py: this build runs on one GPU only; run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if opt.traffic_from:
        return write_traffic_record(*opt.traffic_from)
    NODES = opt.tree_tokens
    if opt.loop:
        if opt.steps == 50:
            opt.steps = 300
        print(json.dumps(loop_bench(opt)), flush=True)
        return
    if opt.gemm:
        print(json.dumps(gemm_bench(opt)), flush=True)
        return
    if opt.small_m:
        print(json.dumps(small_m_bench(opt)), flush=True)
        return
    if opt.cpu_qmm:
        print(json.dumps(cpu_qmm_bench(opt)), flush=True)
        return
    if opt.attention:
        print(json.dumps(attention_bench(opt)), flush=True)
        return

    import torch
    from mlx_eagle_spec_decoding_tree_amd import _lib, eagle, llama, ops, synth
    from mlx_eagle_spec_decoding_tree_amd.cache import make_prompt_cache

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    _lib.check(_lib.lib().eagle_check_device(), "device check")

    if opt.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    args = synth.qwen25_7b()
    t0 = time.time()
    weights = synth.make_model_weights(args, seed=opt.seed)
    print(f"[bench] synthetic weights: {sum(v.nbytes for v in weights.values()) / 1e9:.2f} GB "
          f"in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    model = llama.Model.from_numpy(args, weights, dev)
    rng = np.random.default_rng(opt.seed + 1)
    G, hd, L = args.num_key_value_heads, args.head_dim, args.num_hidden_layers
    cap = 4096
    cache = make_prompt_cache(model, capacity=cap)
    prefix = []
    for c in cache:
        k = rng.standard_normal((G, PREFIX, hd), dtype=np.float32).astype(np.float16)
        v = rng.standard_normal((G, PREFIX, hd), dtype=np.float32).astype(np.float16)
        c.keys[0, :, :PREFIX].copy_(torch.from_numpy(k).to(dev))
        c.values[0, :, :PREFIX].copy_(torch.from_numpy(v).to(dev))
        c.offset = PREFIX
        prefix.append((k, v))
    cache[0].sync_len()

    parents = synth.random_tree(rng, NODES)
    depth, anc, bits = synth.tree_arrays(parents)
    tokens = rng.integers(0, args.vocab_size, NODES).astype(np.int32)

    slab_plan = None
    if opt.slabs is not None:
        slab_plan = {kv.split("=")[0]: int(kv.split("=")[1]) for kv in opt.slabs.split(",") if kv}
    ver = eagle.TreeVerifier(model, cache, total_tokens=NODES - 1, max_len=cap, slab_plan=slab_plan)
    ver.set_tree(torch.from_numpy(tokens).to(dev), torch.from_numpy(depth.astype(np.int32)).to(dev),
                 torch.from_numpy(parents).to(dev),
                 torch.from_numpy(bits.view(np.int32)).to(dev))
    len0 = torch.tensor([PREFIX], dtype=torch.int32, device=dev)

    def one_step():
        ver.len_dev.copy_(len0)               # rewind: every step sees the same 2048-token prefix
        ver.forward()

    # A tree of random tokens is rejected at the root.  The draft tokens along one root-to-leaf
    # path are therefore set to what the target itself predicts there (one eager step per level:
    # a node's logits depend on its ancestors' tokens only), so that the timed step accepts a
    # chain of ACCEPT_CHAIN tokens and compacts their K / V rows, as a step of the loop does.
    path = [int(np.argmax(depth))]
    while path[-1] != 0:
        path.append(int(parents[path[-1] - 1]))
    path = path[::-1][:ACCEPT_CHAIN + 1]
    for parent, child in zip(path[:-1], path[1:]):
        one_step()
        tokens[child] = int(ver.node_argmax[parent].item())
        ver.set_tree(torch.from_numpy(tokens).to(dev), torch.from_numpy(depth.astype(np.int32)).to(dev),
                     torch.from_numpy(parents).to(dev), torch.from_numpy(bits.view(np.int32)).to(dev))

    # ---- timed region: W warm-up replays, then exactly K replays ----
    _, graph = graph_time_ms(torch, one_step, reps=1, warm=0)
    for _ in range(opt.warmup):
        graph.replay()
    torch.cuda.synchronize()
    t_start = time.perf_counter()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(opt.steps):
        graph.replay()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t_start) * 1e3 / opt.steps
    ms_per_step = e0.elapsed_time(e1) / opt.steps
    result = ver.result.cpu().numpy().copy()
    gpu_logits = ver.logits.cpu().numpy().copy()

    # ---- dominant kernel: the QMM launches of one step, replayed alone ----
    launches = ver.qmm_launches()
    ver.hn.normal_()
    ver.attn.normal_()
    ver.act.normal_()

    def qmm_only(subset=None):
        for wq, sc, bi, bias, x, out, form, tiled in (launches if subset is None else subset):
            if form is True:
                ops.quantized_matmul_swiglu(x, wq, sc, bi, bias=bias, out=out, tiled=tiled)
            elif form == "rows":
                ops.quantized_matmul_tiled(x, tiled, bias=bias, out=out)
            elif form:
                ops.quantized_matmul_slabs(x, wq, sc, bi, form, partial=ver.partial, tiled=tiled)
            else:
                ops.quantized_matmul(x, wq, sc, bi, bias=bias, out=out)

    def alg_bytes(l):
        return qmm_bytes(NODES, l[0].shape[0], l[0].shape[1] * 8, l[5].shape[-1])

    qt, _ = graph_time_ms(torch, qmm_only, reps=10)
    qmm_ms = float(np.median(qt))
    n_launch = len(launches)
    alg = sum(alg_bytes(l) for l in launches)
    kv_bytes = 2 * L * G * (PREFIX + NODES) * hd * 2
    achieved = alg / (qmm_ms * 1e-3) / 1e9
    traffic, traffic_source = read_traffic_record()
    stream_kernel = "qmm_w4g64_kernel"          # (above 32 tree tokens: two launches of it per product)
    burst = (not ver.wide) and any(l[6] is True and l[7] is not None for l in launches)
    rows_form = any(l[6] == "rows" for l in launches)
    kernels = ((stream_kernel if any(not l[6] for l in launches) else "qmm_rows_tiled_kernel")
               + " + qmm_slab_w4g64_kernel" + (" + qmm_burst_w4g64_kernel" if burst else "")
               + (" + qmm_rows_tiled_kernel" if rows_form and any(not l[6] for l in launches) else ""))
    roofline = {"bound": "hbm", "kernel": kernels, "achieved": round(achieved, 1),
                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                "traffic": traffic, "traffic_source": traffic_source, "launches_per_step": n_launch,
                "avg_launch_us": round(qmm_ms * 1e3 / n_launch, 3),
                "algorithmic_bytes_per_launch": round(alg / n_launch),
                "step_frac": round((alg + kv_bytes) / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}

    # the same for each kernel on its own launches
    per_kernel = {}
    # (above 32 tree tokens gate|up + SwiGLU runs on the slab kernel too: one slab over all of K)
    swi_on_slab = ver.wide or any(l[6] is True and l[7] is not None for l in launches)
    swi_name = ("qmm_burst_w4g64_kernel (gate|up + SwiGLU)" if burst else
                "qmm_slab_w4g64_kernel (SwiGLU form)" if swi_on_slab else stream_kernel)
    groups = ([(swi_name, [l for l in launches if l[6] is True]), (stream_kernel, [l for l in launches if not l[6]])]
              if swi_on_slab else [(stream_kernel, [l for l in launches if l[6] is True or not l[6]])])
    for kname, sub in (*groups,
                       ("qmm_rows_tiled_kernel (vocabulary projection)", [l for l in launches if l[6] == "rows"]),
                       ("qmm_slab_w4g64_kernel", [l for l in launches if l[6] and l[6] is not True and l[6] != "rows"])):
        if not sub:
            continue
        st, _ = graph_time_ms(torch, lambda: qmm_only(sub), reps=10)
        sub_ms = float(np.median(st))
        sub_alg = sum(alg_bytes(l) for l in sub)
        per_kernel[kname] = {"launches_per_step": len(sub), "avg_launch_us": round(sub_ms * 1e3 / len(sub), 3),
                             "algorithmic_bytes_per_launch": round(sub_alg / len(sub)),
                             "achieved": round(sub_alg / (sub_ms * 1e-3) / 1e9, 1),
                             "frac": round(sub_alg / (sub_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
    roofline["per_kernel"] = per_kernel

    if opt.sweep:
        sweep(torch, ops, dev, args)

    # ---- CPU baseline: the CPU restatement of the same step on the host cores, same inputs ----
    cpu = None
    parity = None
    if not opt.no_cpu:
        from oracle import model_oracle, oracle
        oracle.build()
        have = os.cpu_count() or 1
        cores = int(os.environ.get("OMP_NUM_THREADS", 0)) or min(16, have)
        inv, sc = synth.inv_freqs(args)

        def cpu_step(layers=None):
            oc = model_oracle.new_cache(args, PREFIX + NODES, layers)
            for (ok, ov), (k, v) in zip(oc, prefix):
                ok[:, :PREFIX] = k
                ov[:, :PREFIX] = v
            t0 = time.perf_counter()
            out = model_oracle.verify_step(args, weights, inv, sc, tokens, depth, parents, anc, oc, PREFIX,
                                           layers=layers)
            return out, (time.perf_counter() - t0) * 1e3

        print(f"[bench] CPU baseline: full steps on {cores} host threads ...", file=sys.stderr, flush=True)
        set_omp_threads(cores)
        cpu_step()                                      # warm-up: pages in the 4.3 GB of weights
        cpu_runs = [cpu_step() for _ in range(3)]
        want = cpu_runs[0][0]
        cpu_ms = float(np.median([t for _, t in cpu_runs]))
        # one thread: a step of 1 layer and a step of 3 layers (+ embedding, head, acceptance);
        # the difference prices a layer, the full step is extrapolated from it
        print("[bench] CPU baseline: 1-layer and 3-layer steps on one host thread ...", file=sys.stderr, flush=True)
        set_omp_threads(1)
        _, t1 = cpu_step(1)
        _, t3 = cpu_step(3)
        set_omp_threads(cores)
        single_est = t1 + (L - 1) * (t3 - t1) / 2.0
        cpu = {"value": round(cpu_ms, 1), "unit": "ms", "cores": cores, "cores_available": have,
               "cpu_model": cpu_model(), "kind": "port",
               "sample": "1 full step (28 layers + head, 32 nodes, 2048-token prefix), same weights and inputs, "
                         "OpenMP C restatement, median of 3 timed steps after one warm-up step",
               "runs_ms": [round(t, 1) for _, t in cpu_runs],
               "single_thread": {"value": round(single_est, 1), "unit": "ms", "cores": 1,
                                 "measured": {"one_layer_step_ms": round(t1, 1), "three_layer_step_ms": round(t3, 1)},
                                 "sample": "measured on one thread: a 1-layer step and a 3-layer step (both with "
                                           "embedding, head and acceptance); `value` extrapolates them to 28 layers"}}
        wl = want["logits"].astype(np.float32)
        gl = gpu_logits.astype(np.float32)
        abs_err = float(np.abs(gl - wl).max())
        err = abs_err / float(np.sqrt(np.mean(wl * wl)))
        srt = np.sort(wl, axis=-1)
        clear = (srt[:, -1] - srt[:, -2]) > 2 * abs_err       # nodes whose top-2 margin exceeds the error
        am_gpu = np.argmax(gl, -1)
        parity = {"finite": bool(np.isfinite(gl).all() and np.isfinite(wl).all()),
                  "logits_max_abs_err_over_rms": round(err, 5), "per_operator_tolerance": 2e-2,
                  "full_depth_bound": FULL_DEPTH_BOUND,
                  "node_argmax_equal": int((am_gpu == want["node_argmax"]).sum()),
                  "nodes_with_clear_margin": int(clear.sum()),
                  "clear_margin_argmax_equal": int((am_gpu[clear] == want["node_argmax"][clear]).sum()),
                  "nodes": NODES,
                  "accept_length": int(result[1]), "accept_length_cpu": int(want["accept_length"]),
                  "accept_equal": bool(result[0] == want["best"] and result[1] == want["accept_length"]
                                       and result[3] == want["next_token"])}
        parity["ok"] = bool(parity["finite"] and err <= FULL_DEPTH_BOUND and parity["accept_equal"]
                            and parity["clear_margin_argmax_equal"] == parity["nodes_with_clear_margin"])

    line = {"metric": "tree_verify_step_ms", "value": round(ms_per_step, 4), "unit": "ms", "n_gpus": 1,
            "steps": opt.steps, "warmup": opt.warmup, "ms_per_step": round(ms_per_step, 4),
            "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
            "data": "synthetic",
            "config": {"workload": f"qwen2.5-7b-shape 4-bit g64 target, 28 layers, {NODES} tree nodes, "
                                   "2048-token fp16 KV prefix, greedy accept + KV compaction, HIP-graph replay",
                       "nodes": NODES, "prefix": PREFIX, "wall_ms_per_step": round(wall_ms, 4),
                       "accept_length": int(result[1]),
                       "tokens_per_target_forward": int(result[1]) + 1},
            "roofline": roofline, "cpu_baseline": cpu}
    if parity is not None:
        line["parity"] = parity
    if not opt.headline_only:
        # the other workloads, driver-timed in the same run (their own keys; the headline keys
        # above are untouched)
        if NODES <= 32:
            # the same step on a tree of the reference's default size (39 draft nodes, mlx_eagle.py:390,510)
            wt = 40
            wparents = synth.random_tree(rng, wt)
            wdepth, _, wbits = synth.tree_arrays(wparents)
            wver = eagle.TreeVerifier(model, cache, total_tokens=wt - 1, max_len=cap)
            wver.set_tree(torch.from_numpy(rng.integers(0, args.vocab_size, wt).astype(np.int32)).to(dev),
                          torch.from_numpy(wdepth.astype(np.int32)).to(dev), torch.from_numpy(wparents).to(dev),
                          torch.from_numpy(wbits.view(np.int32)).to(dev))

            def wide_step():
                wver.len_dev.copy_(len0)
                wver.forward()

            wt_ms, wgraph = graph_time_ms(torch, wide_step, reps=20)
            line["wide_tree"] = {"metric": "tree_verify_step_ms at the reference's default tree size",
                                 "tree_tokens": wt, "value": round(float(np.median(wt_ms)), 4), "unit": "ms",
                                 "steps": 20}
            del wver, wgraph
        del ver, graph, model, cache, weights
        torch.cuda.empty_cache()
        extra = argparse.Namespace(**vars(opt))
        extra.steps, extra.warmup, extra.self_draft = 50, 3, False
        extra.depth, extra.draft_nodes = 3, 31
        lp = loop_bench(extra)
        line["loop"] = {k: lp[k] for k in ("metric", "value", "unit", "steps", "ms_per_step", "tokens_per_step",
                                           "prefill_ms", "parity")}
        line["loop"]["workload"] = lp["config"]["workload"]
        torch.cuda.empty_cache()
        line["qmm_sweep"] = qmm_sweep(torch, ops, dev, with_cpu=not opt.no_cpu)
        extra.steps, extra.warmup = 10, 2
        gm = gemm_bench(extra)
        line["prompt_gemm"] = {"metric": gm["metric"], "value": gm["value"], "unit": gm["unit"],
                               "frac_of_mfma_peak": gm["roofline"]["frac"], "shapes": gm["shapes"],
                               "workload": gm["config"]["workload"]}
    print(json.dumps(line), flush=True)
    if parity is not None and not parity["ok"]:
        print("bench.py: full-size parity check failed (see `parity` in the line above)", file=sys.stderr)
        sys.exit(1)


def gemm_bench(opt):
    """The linear layers of one Llama-3-8B-shaped decoder layer over a 512-row prompt chunk
    (mlx_eagle.py:522-533): tiled MFMA GEMM with in-register dequantisation.  Bound by the matrix
    cores: 2*M*N*K flops per launch against 2.5 PFLOP/s dense fp16."""
    import torch
    from mlx_eagle_spec_decoding_tree_amd import _lib, ops

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    _lib.check(_lib.lib().eagle_check_device(), "device check")
    M = 512
    shapes = [("q|k|v", 6144, 4096), ("o", 4096, 4096), ("gate|up", 28672, 4096), ("down", 4096, 14336)]
    gen = torch.Generator(device=dev).manual_seed(opt.seed)
    rows, total_us, total_flop = [], 0.0, 0.0
    for name, N, K in shapes:
        w = torch.randint(-2 ** 31, 2 ** 31 - 1, (N, K // 8), dtype=torch.int32, device=dev, generator=gen)
        sc = (torch.rand(N, K // 64, device=dev, generator=gen) * 0.015 + 0.005).half()
        bi = (-8 * sc.float()).half()
        x = torch.randn(M, K, device=dev, generator=gen).half()
        out = torch.empty(M, N, dtype=torch.float16, device=dev)
        ms, _ = graph_time_ms(torch, lambda: ops.quantized_matmul(x, w, sc, bi, out=out), opt.steps, opt.warmup)
        us = 1e3 * sorted(ms)[len(ms) // 2]
        flop = 2.0 * M * N * K
        rows.append({"name": name, "N": N, "K": K, "us": round(us, 2), "tflops": round(flop / us / 1e6, 1)})
        total_us += us
        total_flop += flop
    achieved = total_flop / total_us / 1e6
    line = {
        "metric": "prompt-pass quantised matmul, TFLOP/s over the linear layers of one decoder layer",
        "value": round(achieved, 1), "unit": "TFLOP/s", "n_gpus": 1, "steps": opt.steps, "warmup": opt.warmup,
        "ms_per_step": round(total_us / 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "Llama-3-8B-shaped 4-bit g64 layer, 512-row prompt chunk: q|k|v, o, gate|up, "
                               "down as tiled MFMA GEMMs", "rows": M},
        "roofline": {"bound": "mfma", "kernel": "qmm_gemm_w4g64_kernel", "achieved": round(achieved, 1),
                     "peak": 2500.0, "unit": "TFLOP/s", "frac": round(achieved / 2500.0, 4), "traffic": None},
        "shapes": rows,
    }
    return line


def attention_bench(opt):
    """Tree-position RoPE with the cache append, then tree-masked GQA attention, as the step
    launches them per layer: 32 tree tokens (seeded random tree, depth <= 4), 28 query / 4 KV
    heads of 128, fp16 KV prefix of P tokens.  28 caches in rotation (one per layer of the 7B
    shape), graph-timed; bytes = the K and V rows read (2 * 4 * (P + 32) * 128 * 2)."""
    import torch
    from mlx_eagle_spec_decoding_tree_amd import _lib, ops, synth

    dev = torch.device("cuda:0")
    _lib.check(_lib.lib().eagle_check_device(), "device check")
    H, G, hd, T, layers = 28, 4, 128, 32, 28
    rng = np.random.default_rng(opt.seed)
    parents = synth.random_tree(rng, T)
    depth, anc, bits = synth.tree_arrays(parents)
    bits_d = torch.from_numpy(bits.view(np.int32)).to(dev)
    inv = ops.default_inv_freqs(hd, 1e6, dev)
    rows = []
    for P in (1024, 2048):
        cap = P + 64
        K = [torch.randn(G, cap, hd, device=dev).half() for _ in range(layers)]
        V = [torch.randn(G, cap, hd, device=dev).half() for _ in range(layers)]
        qkv = torch.randn(T, (H + 2 * G) * hd, device=dev).half()
        pos = (torch.from_numpy(depth.astype(np.int32)).to(dev) + P).contiguous()
        len_dev = torch.tensor([P], dtype=torch.int32, device=dev)
        cs = ops.rope_table(pos, inv, 1.0)
        q_rot = torch.empty(H, T, hd, device=dev, dtype=torch.float16)
        out = torch.empty(T, H * hd, device=dev, dtype=torch.float16)
        ops.workspace("attn", _lib.lib().eagle_tree_attention_workspace_bytes(H, hd, cap), dev)

        def rope():
            for i in range(layers):
                ops.rope_kv_append(qkv, qkv[:, H * hd:], qkv[:, (H + G) * hd:], pos, inv, 1.0, q_rot, K[i], V[i],
                                   len_dev, H, G, hd, row_stride=(H + 2 * G) * hd, rope_cs=cs)

        def attn():
            for i in range(layers):
                ops.tree_attention(q_rot, K[i], V[i], bits_d, len_dev, hd ** -0.5, max_len=cap, out=out)

        def both():
            for i in range(layers):
                ops.rope_kv_append(qkv, qkv[:, H * hd:], qkv[:, (H + G) * hd:], pos, inv, 1.0, q_rot, K[i], V[i],
                                   len_dev, H, G, hd, row_stride=(H + 2 * G) * hd, rope_cs=cs)
                ops.tree_attention(q_rot, K[i], V[i], bits_d, len_dev, hd ** -0.5, max_len=cap, out=out)

        t = {n: float(np.median(graph_time_ms(torch, f, reps=7)[0])) * 1e3 / layers
             for n, f in (("rope_append_us", rope), ("attention_us", attn), ("both_us", both))}
        kv = 2 * G * (P + T) * hd * 2
        rows.append({"prefix": P, **{k: round(v, 2) for k, v in t.items()}, "kv_bytes": kv,
                     "attention_frac_of_hbm_peak": round(kv / t["attention_us"] / 1e3 / HBM_PEAK_GBS, 4)})
    # causal attention of a prompt chunk (mlx_llama.py:185-192 with the causal mask of :275-276):
    # all 32-row pieces of the chunk in one launch pair, behind P0 cache rows
    causal = []
    for name, (Hc, Gc, hdc) in (("8B target", (32, 8, 128)), ("7B target", (28, 4, 128)), ("0.5B drafter", (14, 2, 64))):
        for R, P0 in ((512, 0), (512, 1536), (2048, 0)):
            cap = P0 + R + 256
            q = torch.randn(Hc, R, hdc, device=dev).half()
            kc = torch.randn(Gc, cap, hdc, device=dev).half()
            vc = torch.randn(Gc, cap, hdc, device=dev).half()
            out = torch.empty(R, Hc * hdc, device=dev, dtype=torch.float16)
            piece_len = torch.tensor([P0 + 32 * j for j in range(R // 32)], dtype=torch.int32, device=dev)
            ops.causal_attention(q, kc, vc, piece_len, hdc ** -0.5, max_len=cap, out=out)

            def chunk():
                for _ in range(8):
                    ops.causal_attention(q, kc, vc, piece_len, hdc ** -0.5, max_len=cap, out=out)

            us = float(np.median(graph_time_ms(torch, chunk, reps=7)[0])) * 1e3 / 8
            keys = sum(P0 + 32 * j + 32 for j in range(R // 32))
            flops = 4.0 * Hc * 32 * keys * hdc          # S and O products over the keys each piece sees
            causal.append({"shape": name, "rows": R, "cache_rows": P0, "us": round(us, 2),
                           "tflops": round(flops / us / 1e6, 1)})
            del q, kc, vc, out
    return {"metric": "tree-position rope + tree-masked attention, us per layer", "unit": "us", "dtype": "f16",
            "data": "synthetic", "config": {"workload": "32 tree tokens, 28 q / 4 kv heads, head_dim 128, theta 1e6"},
            "rows": rows, "causal_chunk": causal}


def cpu_qmm_bench(opt):
    """The CPU restatement of one quantised matmul (oracle/eagle_oracle.c, OpenMP) on the host
    cores: median of the timed calls after the warm-up calls (10 + 20 for the small shapes, as the
    reference's own timing loop drops 10 of 30, utils.py:59-72; 3 + 7 for the 300 MB vocabulary
    projection), with all threads and with one."""
    from mlx_eagle_spec_decoding_tree_amd import synth
    from oracle import oracle
    oracle.build()
    have = os.cpu_count() or 1
    cores = int(os.environ.get("OMP_NUM_THREADS", 0)) or min(16, have)
    shapes = [("cfg1", 8192, 2048), ("q/o", 3584, 3584), ("k/v", 512, 3584), ("gate/up", 18944, 3584),
              ("down", 3584, 18944), ("lm_head", 152064, 3584)]
    rng = np.random.default_rng(42)
    rows = []
    for name, N, K in shapes:
        layer = synth.make_qlinear(rng, N, K)
        big = N * K > 2e8
        for M in (1, 8, 16, 24, 32):
            x = synth.make_x(rng, M, K)
            rec = {"name": name, "N": N, "K": K, "M": M}
            for label, threads in (("all_threads_us", cores), ("one_thread_us", 1)):
                if label == "one_thread_us" and (big or M not in (8, 32)):
                    continue
                set_omp_threads(threads)
                warm, timed = (3, 7) if big else ((10, 20) if threads > 1 else (3, 7))
                ts = []
                for it in range(warm + timed):
                    t0 = time.perf_counter()
                    oracle.qmm(x, layer["weight"], layer["scales"], layer["biases"])
                    if it >= warm:
                        ts.append((time.perf_counter() - t0) * 1e6)
                rec[label] = round(float(np.median(ts)), 1)
            rows.append(rec)
            print(f"[cpu-qmm] {rec}", file=sys.stderr, flush=True)
    set_omp_threads(cores)
    return {"metric": "CPU restatement of one quantised matmul, us per call (median)", "unit": "us",
            "cores": cores, "cores_available": have, "cpu_model": cpu_model(), "kind": "port", "rows": rows}


def small_m_bench(opt):
    """M in {1, 2, 4, 8} over the projection shapes of the Qwen2.5-7B-shaped model:
    eagle_qmv_rows_w4g64_f16 (v_dot2_f32_f16 + DPP row sums, the expanded nibbles shared by the rows)
    beside eagle_qmm_w4g64_f16 (16-row MFMA tiles with the other rows idle), each launch on its own
    copy of the weights (> 1 GB in rotation)."""
    import torch
    from mlx_eagle_spec_decoding_tree_amd import _lib, ops

    dev = torch.device("cuda:0")
    _lib.check(_lib.lib().eagle_check_device(), "device check")
    L = _lib.lib()
    shapes = [("q/o", 3584, 3584), ("k/v", 512, 3584), ("gate/up", 18944, 3584), ("down", 3584, 18944),
              ("lm_head", 152064, 3584), ("cfg1", 8192, 2048)]
    rows = []
    st = lambda: torch.cuda.current_stream().cuda_stream
    for name, N, K in shapes:
        ncopy = max(2, min(16, (1 << 30) // (N * K // 2)))
        ws = [torch.randint(-2 ** 31, 2 ** 31 - 1, (N, K // 8), dtype=torch.int32, device=dev) for _ in range(ncopy)]
        ss = [(torch.rand(N, K // 64, device=dev) * 0.015 + 0.005).half() for _ in range(ncopy)]
        bs = [(-8 * s.float()).half() for s in ss]
        for M in (1, 2, 4, 8):
            x = torch.randn(M, K, device=dev).half()
            o = torch.empty(M, N, device=dev, dtype=torch.float16)
            wsp = ops.workspace("qmm", L.eagle_qmm_workspace_bytes(M, N, K), dev)
            iters = 24

            def mfma():
                for i in range(iters):
                    j = i % ncopy
                    _lib.check(L.eagle_qmm_w4g64_f16(x.data_ptr(), ws[j].data_ptr(), ss[j].data_ptr(), bs[j].data_ptr(),
                                                     None, o.data_ptr(), M, N, K, 64, 4, wsp.data_ptr(), wsp.numel(),
                                                     st()), "qmm")

            def valu():
                for i in range(iters):
                    j = i % ncopy
                    _lib.check(L.eagle_qmv_rows_w4g64_f16(x.data_ptr(), ws[j].data_ptr(), ss[j].data_ptr(),
                                                          bs[j].data_ptr(), None, o.data_ptr(), M, N, K, 64, 4, st()),
                               "qmv")

            t_m = float(np.median(graph_time_ms(torch, mfma, reps=7)[0])) * 1e3 / iters
            rec = {"name": name, "N": N, "K": K, "M": M, "mfma_us": round(t_m, 2)}
            byts = qmm_bytes(M, N, K)
            rec["mfma_frac"] = round(byts / t_m / 1e3 / HBM_PEAK_GBS, 4)
            if L.eagle_qmv_rows_supported(M, N, K):
                t_v = float(np.median(graph_time_ms(torch, valu, reps=7)[0])) * 1e3 / iters
                rec["valu_us"] = round(t_v, 2)
                rec["valu_frac"] = round(byts / t_v / 1e3 / HBM_PEAK_GBS, 4)
            rec["dispatched_to"] = "valu" if ops.qmv_preferred(N, K, M) else "mfma"
            rows.append(rec)
            print(f"[small-m] {rec}", file=sys.stderr, flush=True)
        del ws, ss, bs
    return {"metric": "quantised product of 1..8 rows, us per launch (vector ALU beside matrix tiles)", "unit": "us",
            "dtype": "f16", "data": "synthetic", "rows": rows}


def loop_bench(opt):
    """End-to-end greedy tree loop (mlx_eagle.py:503-606) on synthetic models."""
    import torch
    from mlx_eagle_spec_decoding_tree_amd import _lib, llama, ops, spec, synth

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    _lib.check(_lib.lib().eagle_check_device(), "device check")
    steps = opt.steps
    k, depth, nodes, prompt_len = 8, opt.depth, opt.draft_nodes, 512
    targs = synth.llama3_8b()
    t0 = time.time()
    target = llama.Model.from_numpy(targs, synth.make_model_weights(targs, seed=opt.seed), dev)
    if opt.self_draft:
        dargs = targs
        draft = llama.Model.from_numpy(targs, synth.make_model_weights(targs, seed=opt.seed), dev)
    else:
        dargs = synth.qwen25_05b()
        draft = llama.Model.from_numpy(dargs, synth.make_model_weights(dargs, seed=opt.seed + 1), dev)
    print(f"[bench] synthetic models in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    rng = np.random.default_rng(opt.seed + 2)
    prompt = torch.from_numpy(rng.integers(0, min(targs.vocab_size, dargs.vocab_size), prompt_len)).to(dev)
    capacity = prompt_len + (opt.warmup + steps) * (depth + 2) + k * depth + 64
    plans = [None if s is None else {kv.split("=")[0]: int(kv.split("=")[1]) for kv in s.split(",") if kv}
             for s in (opt.slabs, opt.draft_slabs)]
    dec = spec.SpeculativeDecoder(target, draft, capacity=capacity, k=k, depth=depth,
                                  verify_num_tokens=nodes, max_out=(opt.warmup + steps) * (depth + 2) + 8,
                                  slab_plan=plans[0], draft_slab_plan=plans[1],
                                  draft_folded=False if opt.no_draft_folded else None)
    dec.prepare(prompt_len)
    torch.cuda.synchronize()
    t0 = time.time()
    dec.prefill(prompt)
    torch.cuda.synchronize()
    prefill_ms = (time.time() - t0) * 1e3
    dec.capture()
    for _ in range(opt.warmup):
        dec.step()
    torch.cuda.synchronize()
    n0 = int(dec.out_count.item())
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.time()
    e0.record()
    for _ in range(steps):
        dec.step()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.time() - t0) * 1e3
    gpu_ms = e0.elapsed_time(e1)
    n = int(dec.out_count.item()) - n0
    ms = max(wall_ms, gpu_ms)
    # full-size parity: whatever was drafted, the emitted stream is the target's own greedy
    # stream.  Checked on its first tokens with plain one-token passes of the target fed with the
    # emitted tokens: each emitted token has to be the argmax there, or within the rounding
    # difference between a verification pass and a one-token pass of it (a near-tie).
    n_check = min(24, int(dec.out_count.item()))
    emitted = [dec.first] + dec.out_tokens[:n_check].tolist()
    from mlx_eagle_spec_decoding_tree_amd.cache import make_prompt_cache
    ref_cache = make_prompt_cache(target, capacity=prompt_len + n_check + 40)
    logits = target(prompt[None], cache=ref_cache)[0, -1].float()
    agree, worst = 0, 0.0
    for tok in emitted:
        worst = max(worst, float(logits.max() - logits[tok]))
        agree += int(ops.argmax_rows(logits.half()[None].contiguous()).item()) == tok
        logits = target(torch.tensor([[tok]], dtype=torch.int64, device=dev), cache=ref_cache)[0, -1].float()
    rms = float(logits.pow(2).mean().sqrt())
    # what a step has to move at least: 1 + depth passes of k rows through the drafter and one pass of
    # the tree's rows through the target, each reading its weights once (K / V rows priced at the
    # prompt's length: the caches grow by a few rows per step)
    step_bytes = (1 + depth) * pass_bytes(dargs, k, prompt_len) + pass_bytes(targs, nodes + 1, prompt_len)
    achieved = step_bytes / (ms / steps * 1e-3) / 1e9
    roofline = {"bound": "hbm", "kernel": f"whole loop step: {1 + depth} drafter passes of {k} rows + one target "
                                          f"pass of {nodes + 1} rows (no single kernel dominates)",
                "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                "algorithmic_bytes_per_step": round(step_bytes),
                "target_pass_bytes": round(pass_bytes(targs, nodes + 1, prompt_len)),
                "drafter_pass_bytes": round(pass_bytes(dargs, k, prompt_len))}
    line = {
        "metric": "end-to-end tree loop, generated tokens per second (greedy)",
        "value": round(n / ms * 1e3, 2), "unit": "tokens/s", "n_gpus": 1, "steps": steps,
        "warmup": opt.warmup, "ms_per_step": round(ms / steps, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": ("tree loop: " + ("target drafts for itself" if opt.self_draft else
                                                 "Qwen2.5-0.5B-shaped 4-bit drafter")
                                + f", Llama-3-8B-shaped 4-bit target, 512-token prompt, k 8, depth {depth}, "
                                  f"{nodes} draft nodes"),
                   "prompt_len": prompt_len, "k": k, "depth": depth, "verify_num_tokens": nodes},
        "tokens": n, "tokens_per_step": round(n / steps, 4), "prefill_ms": round(prefill_ms, 1),
        "gpu_ms_total": round(gpu_ms, 2), "wall_ms_total": round(wall_ms, 2),
        "roofline": roofline,
        "parity": {"checked_tokens": len(emitted), "equal_to_target_greedy_stream": agree,
                   "max_logit_deficit_over_rms": round(worst / max(rms, 1e-9), 5),
                   "stream_equal": agree == len(emitted)},
    }
    return line


def qmm_sweep(torch, ops, dev, with_cpu=True):
    """Per-shape table for the JSON line: the single-matmul configuration (8192 x 2048) and the
    five projection shapes of the 7B-shaped target at M in {1, 8, 16, 24, 32}.  GPU: us per launch
    of `quantized_matmul` (graph-timed, weights rotated over more than 1 GB of copies), and of the
    partial-sum slab form on the tiled weight layout where the verification step uses it (its sum
    is taken by the kernel that reads it); algorithmic GB/s and fraction of 8 TB/s of the faster
    one.  CPU: the OpenMP C restatement on all host threads given to the run, median of 20 calls
    after 10 warm-up calls (the reference's own loop drops 10 of 30, utils.py:59-72)."""
    from mlx_eagle_spec_decoding_tree_amd import synth
    shapes = [("cfg1", 8192, 2048), ("q_o", 3584, 3584), ("k_v", 512, 3584), ("gate_up", 18944, 3584),
              ("down", 3584, 18944), ("lm_head", 152064, 3584)]
    rows = []
    cores = None
    if with_cpu:
        from oracle import oracle
        oracle.build()
        cores = int(os.environ.get("OMP_NUM_THREADS", 0)) or min(16, os.cpu_count() or 1)
        set_omp_threads(cores)
    rng = np.random.default_rng(42)
    for name, N, K in shapes:
        wbytes = 0.5625 * N * K
        ncopy = 4 if wbytes > 3e8 else min(40, max(2, int(1.2e9 // wbytes)))
        ws = [torch.randint(-2 ** 31, 2 ** 31 - 1, (N, K // 8), dtype=torch.int32, device=dev) for _ in range(ncopy)]
        ss = [(torch.rand(N, K // 64, device=dev) * 0.015 + 0.005).half() for _ in range(ncopy)]
        bs = [(-8 * s.float()).half() for s in ss]
        steps = ops.slab_steps(32, N, K)
        tiled = [ops.tile_weights(ws[i], ss[i], bs[i]) for i in range(ncopy)] if steps and ops.tiled_supported(32, N, K) else None
        # the whole-product form on the tiled layout, where the step uses it (the vocabulary projection)
        whole = ([ops.tile_weights(ws[i], ss[i], bs[i]) for i in range(ncopy)]
                 if N >= 65536 and ops.rows_tiled_supported(32, N, K) else None)
        layer = synth.make_qlinear(rng, N, K) if with_cpu else None
        for M in (1, 8, 16, 24, 32):
            x = torch.randn(M, K, device=dev).half()
            o = torch.empty(M, N, device=dev, dtype=torch.float16)
            iters = 40

            def fn():
                for i in range(iters):
                    ops.quantized_matmul(x, ws[i % ncopy], ss[i % ncopy], bs[i % ncopy], out=o)

            ts, g = graph_time_ms(torch, fn, reps=5)
            us = float(np.median(ts)) * 1e3 / iters
            rec = {"shape": name, "N": N, "K": K, "M": M, "gpu_us": round(us, 2)}
            best = us
            if tiled is not None:
                part = torch.empty(ops.slab_count(K, steps) * 32 * N, dtype=torch.float32, device=dev)

                def fn_slab():
                    for i in range(iters):
                        ops.quantized_matmul_slabs(x, ws[i % ncopy], ss[i % ncopy], bs[i % ncopy], steps, partial=part,
                                                   tiled=tiled[i % ncopy])

                ts, g = graph_time_ms(torch, fn_slab, reps=5)
                rec["slab_us"] = round(float(np.median(ts)) * 1e3 / iters, 2)
                best = min(best, rec["slab_us"])
            if whole is not None:
                def fn_whole():
                    for i in range(iters):
                        ops.quantized_matmul_tiled(x, whole[i % ncopy], out=o)

                ts, g = graph_time_ms(torch, fn_whole, reps=5)
                rec["tiled_us"] = round(float(np.median(ts)) * 1e3 / iters, 2)
                best = min(best, rec["tiled_us"])
            gbs = qmm_bytes(M, N, K) / best / 1e3
            rec["gbs"] = round(gbs)
            rec["frac"] = round(gbs / HBM_PEAK_GBS, 3)
            if with_cpu:
                xc = synth.make_x(rng, M, K)
                ts = []
                for it in range(30):
                    t0 = time.perf_counter()
                    oracle.qmm(xc, layer["weight"], layer["scales"], layer["biases"])
                    if it >= 10:
                        ts.append((time.perf_counter() - t0) * 1e6)
                rec["cpu_us"] = round(float(np.median(ts)), 1)
            rows.append(rec)
            del g
        del ws, ss, bs, tiled, whole
        torch.cuda.empty_cache()
    return {"gpu": "us per launch, graph-timed, weights rotated over > 1 GB; slab_us = partial-sum slab form on "
                   "the tiled layout (summed by its reader); tiled_us = whole product from the tiled layout (the "
                   "vocabulary projection's form in the step); gbs / frac: algorithmic bytes over the fastest form",
            "cpu": f"OpenMP C restatement, {cores} threads, median of 20 calls after 10 warm-up calls" if with_cpu else None,
            "rows": rows}


def sweep(torch, ops, dev, args):
    """QMM microbenchmark over the projection shapes, weights rotated over > 1 GB of
    distinct copies so that no replay is served from cache."""
    per_layer, head = qmm_shapes(args)
    D, Hq, Gk, hdim = args.hidden_size, args.num_attention_heads, args.num_key_value_heads, args.head_dim
    shapes = ([("cfg1", 8192, 2048)] + [s for s in per_layer if s[0] in ("q", "k", "gate", "down")]
              + [("q|k|v", (Hq + 2 * Gk) * hdim, D), head])
    print(f"{'shape':>8} {'N':>7} {'K':>6} {'M':>3} {'us':>9} {'GB/s':>8} {'frac':>6}", file=sys.stderr)
    for name, N, K in shapes:
        wbytes = 0.5625 * N * K
        ncopy = 4 if wbytes > 3e8 else min(40, max(2, int(1.2e9 // wbytes)))
        ws = [torch.randint(-2 ** 31, 2 ** 31 - 1, (N, K // 8), dtype=torch.int32, device=dev) for _ in range(ncopy)]
        ss = [(torch.rand(N, K // 64, device=dev) * 0.015 + 0.005).half() for _ in range(ncopy)]
        bs = [(-8 * s.float()).half() for s in ss]
        for M in (1, 8, 16, 24, 32):
            x = torch.randn(M, K, device=dev).half()
            o = torch.empty(M, N, device=dev, dtype=torch.float16)
            iters = 40

            def fn():
                for i in range(iters):
                    ops.quantized_matmul(x, ws[i % ncopy], ss[i % ncopy], bs[i % ncopy], out=o)

            ts, _ = graph_time_ms(torch, fn, reps=5)
            us = float(np.median(ts)) * 1e3 / iters
            gbs = qmm_bytes(M, N, K) / us / 1e3
            line = f"{name:>8} {N:>7} {K:>6} {M:>3} {us:>9.2f} {gbs:>8.0f} {gbs / HBM_PEAK_GBS:>6.3f}"
            steps = ops.slab_steps(M, N, K)
            if steps:
                # the slab form at the library's slab length (partial sums only: their sum is
                # taken by the kernel that reads them)
                part = torch.empty(ops.slab_count(K, steps) * 32 * N, dtype=torch.float32, device=dev)

                def fn_slab():
                    for i in range(iters):
                        ops.quantized_matmul_slabs(x, ws[i % ncopy], ss[i % ncopy], bs[i % ncopy], steps, partial=part)

                ts, _ = graph_time_ms(torch, fn_slab, reps=5)
                us_s = float(np.median(ts)) * 1e3 / iters
                gbs_s = qmm_bytes(M, N, K) / us_s / 1e3
                line += f"   slab form ({steps} steps per slab): {us_s:.2f} us {gbs_s:.0f} GB/s {gbs_s / HBM_PEAK_GBS:.3f}"

                nsl = ops.slab_count(K, steps)

                def fn_auto():            # the slab form and the sum of its slabs as a launch of its own
                    for i in range(iters):
                        ops.quantized_matmul_slabs(x, ws[i % ncopy], ss[i % ncopy], bs[i % ncopy], steps, partial=part)
                        ops.slab_sum(part, nsl, M, N, out=o)

                ts, _ = graph_time_ms(torch, fn_auto, reps=5)
                line += f"   with the sum as a second launch: {float(np.median(ts)) * 1e3 / iters:.2f} us"
            print(line, file=sys.stderr, flush=True)
        del ws, ss, bs


if __name__ == "__main__":
    main()

#!/usr/bin/env python3
"""Decode throughput of the 35B-A3B-shaped NVFP4 synthetic model on one MI355X.

A step is one decode token through the whole per-token loop (48 layers in a 3:1
GDN:attention pattern, 512 experts top-10 + shared, NVFP4 experts, Q8_0 dense) after a
layer-at-a-time prefill of a 5,700-token random-id prompt at ctx 8192.  Weights are
synthetic (seed 0), generated on this machine into a GGUF and uploaded once, so every
input is resident in HBM before the timed region starts.

Prints ONE JSON line: decode tok/s, the HBM roofline of the dominant kernel (algorithmic
bytes / HIP-event time on the launch stream) and of the whole token, and the CPU oracle
timed on this box's host cores on a bounded sample of the same model.
"""
import argparse
import json
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT / "inferred-thoughts_amd"))
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0
INT8_PEAK_TOPS = 5000.0    # dense int8 MFMA, published
FP32_MFMA_PEAK_TFLOPS = 157.3
# Per kernel family of the decode graph, from the committed rocprofv3 summary of this same workload
# (profiles/decode_config5_families.txt: its "@" lines; the file says which commands made it): launches per token,
# average duration in the replayed graph (--kernel-trace), HBM bytes fetched and written per launch (--pmc FETCH_SIZE /
# WRITE_SIZE, scaled by a 256 MiB copy).
FAMILY_PROFILE = ROOT / "profiles" / "decode_config5_families.txt"


def family_profile():
    out = {}
    try:
        for line in FAMILY_PROFILE.read_text().splitlines():
            if not line.startswith("@ "):
                continue
            f = [t.strip() for t in line[2:].split("|")]
            if len(f) != 5 or f[0] == "family":
                continue
            out[f[0]] = {"launches_per_token": float(f[1]), "rocprof_avg_us": float(f[2]), "fetched": float(f[3]),
                         "written": float(f[4])}
    except OSError:
        pass
    return out


def summarize_profile(root_dir):
    """The text kept under profiles/ for the decode graph, from three rocprofv3 runs of `bench.py --decode-only` whose
    output directories sit under `root_dir`: trace/ (--kernel-trace), pmc_FETCH_SIZE/ and pmc_WRITE_SIZE/ (--pmc, with
    --copy-ref, whose 256 MiB device copy calibrates the counters).  Needs no GPU.  Prints the per-kernel table of the
    last 48 replayed tokens (count, average duration, average gap before the launch), the "@" lines that
    family_profile() reads, and one GDN layer, one attention layer and the output head node by node."""
    import collections
    import csv
    import glob
    import re
    steps = 48

    def short(n):
        n = n.replace("itk::(anonymous namespace)::", "").replace("itk::", "").replace("void ", "")
        return re.sub(r"\(.*", "", n)

    def grid_of(r):
        if "Grid_Size" in r:
            return int(r["Grid_Size"])
        return int(r["Grid_Size_X"]) * int(r.get("Grid_Size_Y", 1) or 1) * int(r.get("Grid_Size_Z", 1) or 1)

    def family(name, grid):
        n = short(name)
        if n.startswith("layer_chain_k"):
            return "layer_chain (a run of layers, persistent)"
        if n.startswith("fused_gemv_fast_k"):
            return "lm_head (norm + GEMV)" if grid >= 400000 else "fused_gemv (norm + quantize + dense GEMVs)"
        if n.startswith("moe_glu_fast_k"):
            return "moe_glu (expert gate+up)"
        if n.startswith("moe_down_fast_k"):
            return "matmul_experts (expert down)"
        if n.startswith("gdn_rows_fast_k"):
            return "gdn_rows (l2 norm + delta rule)"
        if n.startswith("attend_decode_k") or n.startswith("attend_merge"):
            return "attend"
        if n.startswith("argmax"):
            return "other"
        return None

    trace = glob.glob(f"{root_dir}/trace/**/*kernel_trace.csv", recursive=True)[0]
    rows = []
    for r in csv.DictReader(open(trace)):
        if not r["Kernel_Name"].startswith("__amd_rocclr"):
            rows.append((int(r["Start_Timestamp"]), int(r["End_Timestamp"]), r["Kernel_Name"], grid_of(r)))
    rows.sort()
    # whole tokens: from just after one output-head launch to the next; the last `steps` of them
    heads = [i for i, r in enumerate(rows) if family(r[2], r[3]) == "lm_head (norm + GEMV)"]
    tail = rows[heads[-steps - 1] + 1:heads[-1] + 1]
    nodes = len(tail) // steps
    fam = collections.defaultdict(lambda: [0, 0.0])
    kern = collections.defaultdict(lambda: [0, 0.0, 0.0])
    gaps = 0.0
    for i, (s0, e0, n, g) in enumerate(tail):
        d = (e0 - s0) / 1e3
        fam[family(n, g)][0] += 1
        fam[family(n, g)][1] += d
        k = kern[(short(n), g)]
        k[0] += 1
        k[1] += d
        if i:
            k[2] += (s0 - tail[i - 1][1]) / 1e3
            gaps += (s0 - tail[i - 1][1]) / 1e3
    span = (tail[-1][1] - tail[0][0]) / 1e3
    print(f"kernel trace: the last {steps} replayed decode tokens, {nodes} graph kernels each")
    print(f"per token: {sum(v[1] for v in fam.values()) / steps:.1f} us inside kernels + {gaps / steps:.1f} us between them "
          f"= {span / steps:.1f} us from first start to last end (under the profiler)")
    print(f"{'kernel':50s} {'grid threads':>12s} {'per token':>9s} {'avg us':>8s} {'avg gap before us':>17s} {'us/token':>9s}")
    for (n, g), (c, d, gap) in sorted(kern.items(), key=lambda kv: -kv[1][1]):
        print(f"{n[:50]:50s} {g:12d} {c / steps:9.2f} {d / c:8.2f} {gap / c:17.2f} {d / steps:9.1f}")
    res, scale = {}, {}
    for c in ("FETCH_SIZE", "WRITE_SIZE"):
        f = glob.glob(f"{root_dir}/pmc_{c}/**/*counter_collection.csv", recursive=True)[0]
        acc = collections.defaultdict(lambda: [0, 0.0])
        copies = []
        for r in csv.DictReader(open(f)):
            if r["Counter_Name"] != c:
                continue
            if r["Kernel_Name"].startswith("__amd_rocclr_copyBuffer") and float(r["Counter_Value"]) > 50000:
                copies.append(float(r["Counter_Value"]))
            k = family(r["Kernel_Name"], grid_of(r))
            if k:
                acc[k][0] += 1
                acc[k][1] += float(r["Counter_Value"])
        res[c] = acc
        scale[c] = 262144.0 / (sum(copies) / len(copies)) if copies else float("nan")
        print(f"{c}: a 256 MiB device copy reads {sum(copies) / max(len(copies), 1):.0f} per dispatch over {len(copies)} "
              f"copies -> x {scale[c]:.3f} to KiB")
    print("\n@ family | launches per token | rocprofv3 avg duration us | fetched bytes per launch | written bytes per launch")
    for k in sorted((k for k in fam if k), key=lambda k: -fam[k][1]):
        c, d = fam[k]
        fb, wb = res["FETCH_SIZE"].get(k, [0, 0.0]), res["WRITE_SIZE"].get(k, [0, 0.0])
        print(f"@ {k} | {c / steps:.2f} | {d / c:.3f} | {fb[1] / max(fb[0], 1) * scale['FETCH_SIZE'] * 1024:.0f} | "
              f"{wb[1] / max(wb[0], 1) * scale['WRITE_SIZE'] * 1024:.0f}")
    # the last token: its third GDN layer, the attention layer after it and the output head, node by node
    last = tail[-nodes:]
    glu = [i for i, r in enumerate(last) if short(r[2]).startswith("moe_down_fast_k")]
    chains = [i for i, r in enumerate(last) if short(r[2]).startswith("layer_chain_k")]
    if len(chains) >= 2:   # with layer chains: one chain, the attention mixer behind it, the next chain, and the output head
        cut = last[chains[0]:chains[1] + 1] + last[chains[-1] + 1:]
    else:
        cut = last[glu[1] + 1:glu[3] + 1] + last[glu[-1] + 1:] if len(glu) >= 4 else last
    print("\nlast replayed token node by node (without chains: layers 2 and 3; with them: the first chain, the attention "
          "mixer behind it and the next chain) and the output head: start offset us, duration us, gap before us, kernel, grid threads")
    t0, prev = last[0][0], None
    for s0, e0, n, g in cut:
        gap = "" if prev is None else f"{(s0 - prev) / 1e3:6.2f}"
        print(f"{(s0 - t0) / 1e3:9.2f} {(e0 - s0) / 1e3:7.2f} {gap:>6s}  {short(n)[:70]} {g}")
        prev = e0


def model_path(args):
    base = Path("/dev/shm") if Path("/dev/shm").is_dir() and os.access("/dev/shm", os.W_OK) else Path("/tmp")
    tag = ("_f32router" if args.router_f32 else "") + ("_nvfp4shared" if args.shared_nvfp4 else "")
    return base / f"inferred_hip_bench_L{args.layers}_s{args.seed}{tag}.gguf"


def config1(ih, ob, seed, tmp_dir):
    """Config 1 beside the headline run: the tiny all-Q8_0 model, 32 random prompt ids, 64 greedy tokens.  The GPU's
    exact mode must give the CPU path's token ids; the CPU path is timed on one thread (the reference's bit-exact
    naive run) and on the spin pool, the GPU in both modes."""
    path = Path(tmp_dir) / f"inferred_hip_config1_seed{seed}.gguf"
    ih.synth_write_gguf(path, ih.tiny_config(seed=seed))
    rng = np.random.default_rng(seed)
    prompt = rng.integers(0, 4096, 32).astype(np.uint32)
    out = {"workload": "4 layers (3 GDN + 1 attention), hidden 512, vocab 4096, 16 experts top-4 + shared, all Q8_0; "
                       "32 prompt ids, 64 greedy tokens"}
    om = ob.Model(path)
    cpu_ids = None
    for name, threads in (("cpu_naive_1_thread", 1), ("cpu_spin", min(16, os.cpu_count() or 1))):
        ob.lib().orc_set_threads(threads)
        oe = ob.Engine(om, 128)
        oe.forward(prompt[:-1])
        t = time.perf_counter()
        ids, _ = oe.generate(prompt[-1:], 64)
        dt = time.perf_counter() - t
        out[name] = {"decode_tok_s": round(64 / dt, 1), "threads": threads}
        if cpu_ids is not None:
            out["cpu_spin"]["ids_equal_naive"] = bool(np.array_equal(cpu_ids, ids))
        cpu_ids = np.asarray(ids)
        oe.close()
    ob.lib().orc_set_threads(1)
    om.close()
    for mode, exact in (("gpu_exact", True), ("gpu_fast", False)):
        be = ih.Hip(exact=exact)
        model = ih.Model(path)
        eng = ih.Engine(model, be, 256, 64)
        eng.generate(prompt, 8)      # upload, buffer sizes, graph capture
        eng.reset()
        t = time.perf_counter()
        eng.prefill(prompt, want_logits=False)
        be.sync()
        t_pre = time.perf_counter() - t
        t = time.perf_counter()
        ids = eng.decode_greedy(64)   # device-fed: one wait at the end
        be.sync()
        dt = time.perf_counter() - t
        out[mode] = {"decode_tok_s": round(64 / dt, 1), "prefill_32_ms": round(1e3 * t_pre, 3),
                     "ids_equal_cpu": bool(np.array_equal(cpu_ids, np.asarray(ids)))}
        err = be.take_error()
        if err:
            raise SystemExit(f"device error in the config 1 run: {err}")
        eng.close(); model.close(); be.close()
    try:
        path.unlink()
    except OSError:
        pass
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256, help="greedy decode tokens timed (the baseline workload decodes 256)")
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--layers", type=int, default=48, help="48 is the baseline config; fewer only for quick checks")
    ap.add_argument("--prompt", type=int, default=5700)
    ap.add_argument("--router-f32", action="store_true",
                    help="router, shared-expert gate and ssm alpha / beta matrices in F32 (as real files keep them) "
                         "instead of the baseline's Q8_0: a variant, not the baseline workload")
    ap.add_argument("--shared-nvfp4", action="store_true",
                    help="the shared expert's three matrices in NVFP4 with a second scale each (as an NVFP4 file of this "
                         "model stores them) instead of the baseline's Q8_0: a variant; with --router-f32 it is the "
                         "layout of a real file")
    ap.add_argument("--ctx", type=int, default=8192)
    ap.add_argument("--max-batch", type=int, default=8192,
                    help="tokens per prefill pass; the default takes the 5,700-token prompt through each layer in one "
                         "pass (layer-at-a-time prefill); the reference's own default is 512")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU oracle baseline")
    ap.add_argument("--exact", action="store_true", help="CPU-order reductions (bit-exact mode)")
    ap.add_argument("--keep", action="store_true", help="keep the generated GGUF")
    ap.add_argument("--no-single-ops", action="store_true",
                    help="skip the single-op configurations (expert FFN sweep, decode attention, Gated DeltaNet)")
    ap.add_argument("--decode-only", action="store_true",
                    help="stop after the timed decode stretch (no per-kernel events, no second prefill, no CPU leg): the "
                         "run to put under rocprofv3 --kernel-trace, whose last steps x graph-kernels records are then "
                         "the replayed decode graph and nothing else")
    ap.add_argument("--no-exact-check", action="store_true",
                    help="skip the exact-mode run of the same model (512-token prompt + 32 greedy ids) that the fast "
                         "mode's ids are compared with")
    ap.add_argument("--copy-ref", action="store_true",
                    help="also run one 256 MiB device-to-device torch copy: the kernel of known traffic that "
                         "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE readings are scaled by")
    ap.add_argument("--single-ops-only", action="store_true",
                    help="no model: run the single-op configurations (expert FFN sweep, decode attention, Gated DeltaNet) and "
                         "print their JSON (for rocprofv3 traces of those kernels)")
    ap.add_argument("--ffn-tokens", type=str, default="",
                    help="with --single-ops-only: only the expert FFN, at these token counts (comma-separated)")
    ap.add_argument("--expert-slots", type=int, default=0,
                    help="variant run: fix the expert pool's device tier at this many expert matrices; the rest of the pool "
                         "goes to pinned host memory that the kernels read in place (with --decode-only: prints the tier's "
                         "counters, exchanges experts by the counts of the timed stretch and times a second stretch)")
    ap.add_argument("--expert-host-slots", type=int, default=-1,
                    help="with --expert-slots: cap the pinned host tier at this many expert matrices; what fits neither tier "
                         "is cold and fetched from the model file when a layer picks it (0 = no host tier)")
    ap.add_argument("--no-prefetch", action="store_true",
                    help="with a cold tier: do not read the next layer's likely experts ahead (set_prefetch off)")
    ap.add_argument("--summarize-profile", metavar="DIR",
                    help="no run: print the profiles/ summary of the rocprofv3 outputs under DIR (trace/, pmc_FETCH_SIZE/, "
                         "pmc_WRITE_SIZE/ of --decode-only runs) and exit")
    args = ap.parse_args()
    if args.summarize_profile:
        summarize_profile(args.summarize_profile)
        return
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the path has no collective: experts, layers or heads "
              "would shard across GPUs, none of which is built); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import inferred_hip as ih
    if args.single_ops_only:
        from inferred_hip import single_ops
        ffn = [int(t) for t in args.ffn_tokens.split(",") if t]
        print(json.dumps({"single_op": single_ops.run(ih, seed=args.seed, exact=args.exact, ffn_tokens=ffn)}), flush=True)
        return
    import torch

    t0 = time.time()
    path = model_path(args)
    cfg = ih.big_config(seed=args.seed, n_layer=args.layers, n_threads=min(16, os.cpu_count() or 8))
    if args.router_f32:
        cfg.router_type = ih.ROUTER_F32
    if args.shared_nvfp4:
        cfg.shared_type = ih.NVFP4
    if not path.exists():
        ih.synth_write_gguf(path, cfg)
    t_synth = time.time() - t0
    print(f"[bench] model {path} ({path.stat().st_size / 2**30:.1f} GiB) ready in {t_synth:.1f}s", file=sys.stderr, flush=True)

    if args.copy_ref:
        src = torch.ones(64 << 20, dtype=torch.float32, device="cuda:0")
        dst = torch.empty_like(src)
        dst.copy_(src); torch.cuda.synchronize()
        dst.copy_(src); torch.cuda.synchronize()
        del src, dst
    single = None
    if not args.no_single_ops and args.layers == 48:
        from inferred_hip import single_ops
        t_s = time.time()
        single = single_ops.run(ih, seed=args.seed, exact=args.exact)
        print(f"[bench] single-op configurations in {time.time() - t_s:.1f}s", file=sys.stderr, flush=True)
    be = ih.Hip(exact=args.exact)
    if args.expert_slots:
        be.set_expert_slots(args.expert_slots)
        if args.expert_host_slots >= 0:
            # one repacked expert matrix takes its file bytes (NVFP4: 9 bytes per 16 weights, Q8_0: 34 per 32)
            one = cfg.expert_ff * cfg.n_embd * (9 if cfg.expert_type == ih.NVFP4 else 17) // 16
            be.set_expert_host_budget(max(1, args.expert_host_slots * one))
        be.set_prefetch(not args.no_prefetch)
    model = ih.Model(path)
    eng = ih.Engine(model, be, args.ctx, args.max_batch)
    rng = np.random.default_rng(args.seed)
    prompt = rng.integers(0, model.n_vocab, args.prompt).astype(np.uint32)

    # the first pass uploads and repacks every weight and sizes every device buffer for a full-width pass:
    # charge it to setup, not to prefill
    t1 = time.time()
    eng.forward(prompt[:min(args.prompt, args.max_batch)], want_logits=False)
    be.sync()
    t_upload = time.time() - t1
    eng.reset()
    print(f"[bench] weights resident in {t_upload:.1f}s", file=sys.stderr, flush=True)

    t2 = time.time()
    eng.prefill(prompt, want_logits=False)
    be.sync(); torch.cuda.synchronize()
    t_prefill = time.time() - t2
    print(f"[bench] prefill {args.prompt} tok in {t_prefill:.2f}s", file=sys.stderr, flush=True)

    eng.decode_greedy(args.warmup)
    be.sync(); torch.cuda.synchronize()
    pos0 = eng.pos
    t3 = time.perf_counter()
    ids = eng.decode_greedy(args.steps)
    be.sync(); torch.cuda.synchronize()
    dt = time.perf_counter() - t3
    assert len(ids) == args.steps
    tok_s = args.steps / dt
    graph_stats = be.graph_stats()
    if args.decode_only:
        err = be.take_error()
        if err:
            raise SystemExit(f"device error: {err}")
        line = {"metric": "decode tok/s (decode-only run for a kernel trace)", "value": round(tok_s, 2),
                "unit": "tok/s", "steps": args.steps, "warmup": args.warmup,
                "ms_per_step": round(1e3 * dt / args.steps, 4), "graph": graph_stats}
        if args.expert_slots:
            # the pool's two tiers: where the reads of the run so far were served from, then the same stretch again
            # after the busy host-tier experts have changed places with idle device-tier ones
            st = be.expert_stats()
            t4 = time.perf_counter()
            moved = be.replace_experts_by_counts()
            t_move = time.perf_counter() - t4
            t5 = time.perf_counter()
            eng.decode_greedy(args.steps)
            be.sync()
            dt2 = time.perf_counter() - t5
            st2 = be.expert_stats()
            line["expert_tiers"] = {
                "device_slots": int(st.slots), "host_slots": int(st.host_slots), "slot_bytes": int(st.slot_bytes),
                "reads": int(st.lookups), "reads_from_device_memory": int(st.hits),
                "exchanged_by_counts": int(moved), "exchange_s": round(t_move, 3),
                "tok_s_after_exchange": round(args.steps / dt2, 2),
                "reads_after": int(st2.lookups - st.lookups), "from_device_memory_after": int(st2.hits - st.hits)}
            if st2.oversubscribed:
                tc = be.tier_counters()
                line["expert_tiers"]["cold"] = {
                    "cold_experts": int(st.pool - st.slots - st.host_slots), "fetched": int(tc.fetched),
                    "fetched_in_second_stretch": int(st2.fetched - st.fetched), "fetch_mb": round(tc.fetch_bytes / 1e6, 1),
                    "file_read_ms": round(tc.read_us / 1e3, 1), "upload_issue_ms": round(tc.upload_us / 1e3, 1),
                    "table_writes_ms": round(tc.writes_us / 1e3, 1), "picks_wait_ms": round(tc.picks_wait_us / 1e3, 1),
                    "picks_copy_ms": round(tc.picks_copy_us / 1e3, 1), "prefetch_reads": int(tc.prefetch_reads),
                    "prefetch_used": int(tc.prefetch_used), "prefetch": not args.no_prefetch}
        print(json.dumps(line), flush=True)
        eng.close(); model.close(); be.close()
        if not args.keep:
            try:
                path.unlink()
            except OSError:
                pass
        return
    l0 = be.launch_count(); eng.decode_greedy(1); launches_per_token = be.launch_count() - l0

    # per-kernel device time over a second identical stretch: the launches the decode graph holds, issued
    # one by one on the launch stream with a HIP event before and after each
    be.profile_begin()
    n_prof = min(args.steps, 16)
    eng.decode_greedy(n_prof)
    rows = be.profile_end()
    err = be.take_error()
    if err:
        raise SystemExit(f"device error: {err}")

    n_gdn_layers = sum(1 for il in range(args.layers) if (il + 1) % 4 != 0)
    # per-family device time of one more identical prefill, and the matrix-core rate of each family that uses them
    eng.reset()
    be.profile_begin()
    eng.prefill(prompt, want_logits=False)
    prows = be.profile_end()
    err = be.take_error()
    if err:
        raise SystemExit(f"device error: {err}")
    dense_macs, glu_macs, down_macs = model.token_macs()
    n_attn_layers = args.layers - n_gdn_layers
    F16_PEAK = 2500.0
    # this card's own ceilings: back-to-back MFMA instructions with no memory in the loop, in TOP/s (TFLOP/s)
    ceilings = {kind: round(be.mfma_ceiling(kind) / 1e12, 1) for kind in ih.Hip.MFMA_KINDS}
    # the instruction each family issues
    family_inst = {"matmul (dense": "int8_16x16x32", "moe_glu": "f16_32x32x16", "matmul_experts": "f16_32x32x16",
                   "delta_rule": "f32_16x16x4", "attend": "f16_32x32x16"}
    if args.exact:
        family_inst.update({"moe_glu": "int8_16x16x32", "matmul_experts": "int8_16x16x32"})
    prefill_kernels = {}
    for r in sorted(prows, key=lambda r: -r["ms"]):
        k = {"launches": r["launches"], "ms": round(r["ms"], 2)}
        sec = r["ms"] / 1e3
        if sec <= 0:
            prefill_kernels[r["name"]] = k
            continue
        name = r["name"]
        if name.startswith("matmul (dense"):
            # Q8_0 x Q8_0 on the int8 matrix cores, both modes
            tops = 2 * dense_macs * args.prompt / sec / 1e12
            k.update(unit="int8 MFMA", tops=round(tops, 1), mfma_frac=round(tops / INT8_PEAK_TOPS, 4))
        elif name.startswith("moe_glu") or name.startswith("matmul_experts"):
            m = glu_macs if name.startswith("moe_glu") else down_macs
            useful = 2 * m * args.prompt / sec / 1e12
            if args.exact:
                k.update(unit="int8 MFMA", tops=round(useful, 1), mfma_frac=round(useful / INT8_PEAK_TOPS, 4))
            else:
                # f16 matrix cores, every product issued twice (activation hi and lo halves)
                k.update(unit="f16 MFMA", useful_tops=round(useful, 1), tflops=round(2 * useful, 1),
                         mfma_frac=round(2 * useful / F16_PEAK, 4))
        elif name == "delta_rule" and not args.exact:
            # chunked form, per (64-token chunk, value head): K S^T, Q S^T and the state update (64 x dk x dv each),
            # T R and P U (lower triangles, 64 x 64 x dv / 2 each), K K^T and Q K^T (64 x 64 x dk / 2 each)
            C, dk, dv, heads = 64, 128, 128, 32
            chunk_macs = 3 * C * dk * dv + C * C * dv + C * C * dk
            flops = 2 * chunk_macs * heads * (args.prompt / C) * n_gdn_layers
            k.update(unit="fp32 MFMA", tflops=round(flops / sec / 1e12, 1),
                     mfma_frac=round(flops / sec / 1e12 / FP32_MFMA_PEAK_TFLOPS, 4))
        elif name == "attend" and not args.exact:
            # causal pairs x head_dim x (scores with the query's hi and lo halves + weighted values)
            pairs = args.prompt * (args.prompt + 1) / 2
            flops = 2 * pairs * model.n_head * model.head_dim * 3 * n_attn_layers
            k.update(unit="f16 MFMA", tflops=round(flops / sec / 1e12, 1), mfma_frac=round(flops / sec / 1e12 / F16_PEAK, 4))
        rate = k.get("tflops", k.get("tops"))
        inst = next((v for f, v in family_inst.items() if name.startswith(f)), None)
        if rate is not None and inst is not None:
            k.update(instruction=inst, measured_ceiling=ceilings[inst], frac_of_measured=round(rate / ceilings[inst], 4))
        prefill_kernels[name] = k

    # algorithmic bytes of one decode token (weights once + GDN state r+w + KV read)
    n_attn = sum(1 for il in range(args.layers) if (il + 1) % 4 == 0)
    n_gdn = args.layers - n_attn
    w_bytes = model.decode_weight_bytes()
    state_bytes = n_gdn * 2 * (32 * 128 * 128 * 4) + n_gdn * 2 * (3 * 8192 * 4)
    kv_bytes = n_attn * (pos0 + args.steps // 2) * 512 * 2 * 2
    tok_bytes = w_bytes + state_bytes + kv_bytes
    whole = tok_bytes * tok_s / 1e9

    headline = args.layers == 48 and args.prompt == 5700 and not args.router_f32 and not args.shared_nvfp4 and not args.exact
    rows.sort(key=lambda r: -r["ms"])
    timed = [r for r in rows if r["bytes"]]
    dom = timed[0] if timed else None
    kernels = {r["name"]: {"launches": r["launches"], "ms_per_token": r["ms"] / n_prof,
                           "gb_s": (r["bytes"] / 1e9) / (r["ms"] / 1e3) if r["ms"] > 0 and r["bytes"] else None}
               for r in rows}
    roofline = None
    if dom:
        ach = (dom["bytes"] / 1e9) / (dom["ms"] / 1e3)
        per_launch = dom["bytes"] // dom["launches"]
        prof = family_profile().get(dom["name"]) if headline else None
        # HBM bytes per launch from the committed counter runs.  A reading below the launch's algorithmic bytes cannot
        # be traffic (the weights alone are read once per token and fit no cache): the counters come back short for the
        # 1.4 ms dispatch that holds a whole token, and are then left out (the same layers as thirteen short chains
        # read 1.02 x their algorithmic bytes: profiles/decode_config5_families_attention_between_chains.txt)
        traffic = int(prof["fetched"] + prof["written"]) if prof else None
        traffic_note = None
        if traffic is not None and traffic < 0.8 * per_launch:
            traffic_note = (f"FETCH_SIZE + WRITE_SIZE read {traffic} bytes for this {round(prof['rocprof_avg_us'])} us dispatch, less than "
                            "the weights it must read: counter reading not usable at this dispatch length")
            traffic = None
        roofline = {"bound": "hbm", "kernel": dom["name"], "achieved": round(ach, 1), "peak": HBM_PEAK_GBS,
                    "unit": "GB/s", "frac": round(ach / HBM_PEAK_GBS, 4),
                    "traffic": traffic, "traffic_note": traffic_note,
                    "avg_launch_us": round(1e3 * dom["ms"] / dom["launches"], 2),
                    "bytes_per_launch": per_launch,
                    # the same fraction with the launch duration rocprofv3 reports for this family inside the replayed
                    # graph (no event pair around the launch), from the committed summary
                    "rocprof_avg_launch_us": prof["rocprof_avg_us"] if prof else None,
                    "frac_rocprof": round(per_launch / (prof["rocprof_avg_us"] * 1e-6) / 1e9 / HBM_PEAK_GBS, 4) if prof else None,
                    "profile": str(FAMILY_PROFILE.relative_to(ROOT)) if prof else None}

    # the two arithmetic modes on this very model: a 512-token prompt and 32 greedy ids each.  Exact mode reproduces
    # the CPU path bit for bit (the parity tests); fast mode differs in the last bits, and on random weights, whose
    # logits are nearly tied, a last-bit difference soon picks another token, after which the runs are unrelated.
    mode_check = None
    if not args.exact and not args.no_exact_check:
        n_p, n_g = min(512, args.prompt), 32
        eng.reset()
        lf = eng.prefill(prompt[:n_p])
        ids_fast = np.asarray(eng.decode_greedy(n_g))
        # control: fast mode against ITSELF with the prompt cut into other passes (200 + 200 + rest), which moves the
        # chunk boundaries of the delta rule and the attention kernel's tiles, i.e. last bits only
        eng.reset()
        lc = None
        for at in range(0, n_p, 200):
            lc = eng.forward(prompt[at:min(at + 200, n_p)])
        ids_ctl = np.asarray(eng.decode_greedy(n_g))
        be_x = ih.Hip(exact=True)
        eng_x = ih.Engine(model, be_x, args.ctx, args.max_batch)
        n_h = n_p // 2
        eng_x.prefill(prompt[:n_h], want_logits=False)
        ckpt_half = eng_x.checkpoint()
        eng_x.forward(prompt[n_h:n_p - 1], want_logits=False) if n_p - 1 > n_h else None
        ckpt = eng_x.checkpoint()
        lx = eng_x.forward(prompt[n_p - 1:n_p])
        t_x = time.perf_counter()
        ids_exact = np.asarray(eng_x.decode_greedy(n_g))
        be_x.sync()
        exact_tok_s = n_g / (time.perf_counter() - t_x)
        # Controls with no fast kernel in them, exact mode against exact mode from a checkpoint of its own state:
        #  (a) the state as it was: must reproduce itself bit for bit;
        #  (b) ONE recurrent-state element (the largest) moved by one ulp before the last prompt token;
        #  (c) EVERY recurrent-state element moved by one ulp, up or down at random, half-way through the prompt, the
        #      other half of the prompt run from there: what last-bit noise, the size of a changed summation order,
        #      becomes over 256 tokens of this model.
        eng_x.restore(ckpt)
        l_same = eng_x.forward(prompt[n_p - 1:n_p])
        ids_same = np.asarray(eng_x.decode_greedy(n_g))
        pos_c, conv_c, ssm_c = ckpt
        ssm_u = ssm_c.copy()
        at = int(np.argmax(np.abs(ssm_u)))
        ssm_u[at] = np.nextafter(ssm_u[at], np.float32(np.inf))
        eng_x.restore((pos_c, conv_c, ssm_u))
        l_ulp = eng_x.forward(prompt[n_p - 1:n_p])
        ids_ulp = np.asarray(eng_x.decode_greedy(n_g))
        pos_h, conv_h, ssm_h = ckpt_half
        up = np.random.default_rng(5).random(ssm_h.size) < 0.5
        ssm_n = np.where(up, np.nextafter(ssm_h, np.float32(np.inf)), np.nextafter(ssm_h, np.float32(-np.inf))).astype(np.float32)
        eng_x.restore((pos_h, conv_h, ssm_n))
        l_all = eng_x.forward(prompt[n_h:n_p])
        ids_all = np.asarray(eng_x.decode_greedy(n_g))
        err = be_x.take_error() or be.take_error()
        if err:
            raise SystemExit(f"device error in the mode check: {err}")
        same = ids_fast == ids_exact
        lf64, lx64 = np.asarray(lf, np.float64), np.asarray(lx, np.float64)
        top_x, top_f = np.argsort(-lx64)[:10], np.argsort(-lf64)[:10]
        mode_check = {"prompt": int(n_p), "ids": int(n_g), "ids_equal": int(same.sum()),
                      "equal_prefix": int(np.argmin(same)) if not same.all() else int(n_g),
                      "prefill_logits_max_abs_diff": float(np.abs(lf - lx).max()),
                      "prefill_logits_max_abs": float(np.abs(lx).max()),
                      # how alike the two distributions over the 151,936 tokens are after 512 tokens of prefill
                      "prefill_logits_correlation": round(float(np.corrcoef(lf64, lx64)[0, 1]), 4),
                      "exact_top1_rank_in_fast": int(np.where(np.argsort(-lf64) == top_x[0])[0][0]),
                      "top10_overlap": int(len(set(top_x.tolist()) & set(top_f.tolist()))),
                      "exact_top1_margin": float(lx64[top_x[0]] - lx64[top_x[1]]),
                      "exact_mode_decode_tok_s": round(exact_tok_s, 1),
                      "control_exact_vs_exact_one_ulp": {
                          "what": "exact mode from one checkpoint after 511 prompt tokens: unchanged state, and one "
                                  "recurrent-state element (the largest) moved by one ulp; then the 512th token and 32 greedy ids",
                          "unchanged_state_reproduces_bits": bool(np.array_equal(np.asarray(l_same).view(np.uint32), np.asarray(lx).view(np.uint32))
                                                                  and np.array_equal(ids_same, ids_exact)),
                          "ids_equal": int((ids_ulp == ids_exact).sum()),
                          "logits_max_abs_diff": float(np.abs(np.asarray(l_ulp) - np.asarray(lx)).max()),
                          "logits_correlation": round(float(np.corrcoef(np.asarray(l_ulp, np.float64), lx64)[0, 1]), 6)},
                      "control_exact_vs_exact_every_state_element_one_ulp": {
                          "what": f"exact mode from its own checkpoint after {n_h} prompt tokens, every recurrent-state element "
                                  f"moved by one ulp up or down at random; then the other {n_p - n_h} prompt tokens and 32 greedy ids",
                          "ids_equal": int((ids_all == ids_exact).sum()),
                          "logits_max_abs_diff": float(np.abs(np.asarray(l_all) - np.asarray(lx)).max()),
                          "logits_correlation": round(float(np.corrcoef(np.asarray(l_all, np.float64), lx64)[0, 1]), 6)},
                      "control_fast_vs_fast_other_passes": {
                          "ids_equal": int((ids_ctl == ids_fast).sum()),
                          "prefill_logits_max_abs_diff": float(np.abs(np.asarray(lc) - np.asarray(lf)).max()),
                          "prefill_logits_correlation": round(float(np.corrcoef(np.asarray(lc, np.float64), lf64)[0, 1]), 4)}}
        eng_x.close(); be_x.close()

    cpu = None
    c1 = None
    if not args.no_cpu:
        from oracle import binding as ob
        cores = min(16, os.cpu_count() or 1)
        ob.lib().orc_set_threads(cores)
        om = ob.Model(path)
        oe = ob.Engine(om, 64)
        n_pre, n_dec = 8, 6
        oe.forward(prompt[:n_pre])
        tc = time.perf_counter()
        out, _ = oe.generate(prompt[n_pre:n_pre + 1], n_dec + 1)   # one more pass primes the loop, n_dec decode passes
        dtc = time.perf_counter() - tc
        cpu = {"value": round((n_dec + 1) / dtc, 3), "unit": "tok/s", "cores": cores, "kind": "port",
               "sample": f"{n_dec + 1} single-token passes of the same {args.layers}-layer model at positions "
                         f"{n_pre}..{n_pre + n_dec} (context {n_pre + n_dec}, not 5,700), spin-split rows over {cores} threads"}
        oe.close(); om.close()
        ob.lib().orc_set_threads(1)
        c1 = config1(ih, ob, args.seed, path.parent)

    line = {
        "metric": "decode tok/s & % HBM roofline, 35B-A3B-shape NVFP4 synthetic; prefill tok/s",
        "value": round(tok_s, 2), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(1e3 * dt / args.steps, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "int8 dot / f32 accumulate (NVFP4 + Q8_0 weights, Q8_0 activations)",
        "data": "synthetic",
        "config": {"workload": "config 5: full 35B-A3B-shaped model, greedy decode after a 5,700-token prefill at ctx 8192"
                               if args.layers == 48 and args.prompt == 5700 and not args.router_f32 and not args.shared_nvfp4 else
                               f"VARIANT / reduced check run: {args.layers} layers, prompt {args.prompt}, "
                               f"router {'F32' if args.router_f32 else 'Q8_0'}, shared expert "
                               f"{'NVFP4 with second scales' if args.shared_nvfp4 else 'Q8_0'}",
                   "layers": args.layers, "prompt": args.prompt, "ctx": args.ctx, "prefill_batch": args.max_batch, "decode_pos": int(pos0),
                   "experts": "512 routed experts top-10, NVFP4 with per-expert second scales; one shared expert, " +
                              ("NVFP4 with a second scale per matrix" if args.shared_nvfp4 else "Q8_0"),
                   "dense": "Q8_0 (attention, GDN, LM head; router, shared-gate logit and ssm_alpha/beta Q8_0 too)",
                   "mode": "exact" if args.exact else "fast", "batch": 1},
        "prefill_tok_s": round(args.prompt / t_prefill, 1),
        "prefill_kernels": prefill_kernels,
        "mfma_ceilings_measured": ceilings,
        "single_op": single,
        "bytes_per_token": int(tok_bytes),
        "token_roofline": {"bound": "hbm", "achieved": round(whole, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                           "frac": round(whole / HBM_PEAK_GBS, 4)},
        "roofline": roofline,
        "kernels": kernels,
        "cpu_baseline": cpu,
        "config1": c1,
        "setup_s": {"synth": round(t_synth, 1), "upload_repack": round(t_upload, 1)},
        "graph": graph_stats, "seam_ops_per_token": launches_per_token,
        "exact_vs_fast": mode_check,
    }
    print(json.dumps(line), flush=True)
    eng.close(); model.close(); be.close()
    if not args.keep:
        try:
            path.unlink()
        except OSError:
            pass


if __name__ == "__main__":
    main()

#!/usr/bin/env python3
"""Benchmark of the two KSA attention hot paths on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--prefill-chunks 1024]

Prints ONE JSON line.  A "step" is one prefill forward of a single Summary-Attention
layer on the 128k configuration (1024 chunks x (128 text + 8 summary) rows, 32 query /
8 KV heads, head_dim 128, bf16); `value` is its non-empty-block TFLOP/s.  The decode
attention step over the ring-buffer cache (batch 64, 128k logical context) is timed in a
second region of the same K/W and reported under "decode"; the two smaller prefill configurations, the fused pre-attention step
and the end-to-end decoder of config 4 (batch 8, 32k prompt, 256 greedy steps) follow under their
own keys.  Inputs are synthetic, seeded,
and resident in HBM before any timed region.  The block index is built once before the
timed region (the reference caches it the same way); reading the summary prefix is inside.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBPS = 8000.0      # MI355X HBM3E


def prefill_inputs(chunks, Hq, Hkv, D, C, S, device, seed):
    import torch
    Sq = chunks * (C + S)
    g = torch.Generator(device=device).manual_seed(seed)
    scale = D ** -0.5

    def draw(h):
        t = torch.empty(1, Sq, h, D, dtype=torch.bfloat16, device=device)
        step = 8192
        for r in range(0, Sq, step):
            n = min(step, Sq - r)
            t[0, r:r + n] = (torch.randn(n, h, D, generator=g, device=device) * scale).to(torch.bfloat16)
        return t

    q, k, v = draw(Hq), draw(Hkv), draw(Hkv)
    i = torch.arange(Sq, device=device)
    summary_pos = (i % (C + S)) >= C
    return q, k, v, summary_pos


def time_region(fn, steps, warmup):
    """Runs `warmup` untimed and exactly `steps` timed calls; returns (wall seconds,
    device milliseconds from HIP events recorded on the launch stream)."""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    return t1 - t0, e0.elapsed_time(e1)


def sustained_rate(fn, flop_per_call, seconds, batch):
    """Calls `fn` back to back for `seconds`; returns (TFLOP/s over the second half, mean shader
    clock in MHz over the second half as rocm-smi reports it, or None)."""
    import re
    import subprocess
    import threading
    import torch
    clocks, stop = [], threading.Event()

    def sample():
        while not stop.is_set():
            try:
                r = subprocess.run(["rocm-smi", "-c", "--csv"], capture_output=True, text=True, timeout=5)
                m = re.search(r"\((\d+)Mhz\),\d+\s*$", r.stdout.strip().splitlines()[-1])
                if m:
                    clocks.append((time.perf_counter(), int(m.group(1))))
            except Exception:
                return
            stop.wait(0.2)

    th = threading.Thread(target=sample, daemon=True)
    th.start()
    t0 = time.perf_counter()
    n = n_half = 0
    t_half = None
    while True:
        for _ in range(batch):
            fn()
        torch.cuda.synchronize()
        n += batch
        t = time.perf_counter()
        if t_half is None and t - t0 >= seconds / 2:
            t_half, n_half = t, n
        if t - t0 >= seconds and t_half is not None and n > n_half:
            break
    stop.set()
    th.join()
    late = [c for ts, c in clocks if ts >= t_half]
    return flop_per_call * (n - n_half) / (t - t_half) / 1e12, (sum(late) / len(late) if late else None)


def prefill_record(name, chunks, Hq, Hkv, D, C, S, W, dev, steps, warmup, idle):
    """One prefill configuration timed like the main one: inputs resident, index cached, `steps`
    launches after `warmup`; returns a record with its own roofline object."""
    import torch
    import ksa_amd
    Sq, P = chunks * (C + S), chunks * S
    q, k, v, sp = prefill_inputs(chunks, Hq, Hkv, D, C, S, dev, seed=0)
    idx = ksa_amd.compute_block_sparsity(Sq, Sq + P, C, S, W)
    tiles = int((idx[0] + idx[2]).sum())
    flops = 4.0 * 128 * 64 * D * Hq * tiles

    def step():
        ksa_amd.summary_attn_func(q, k, v, C, S, W, summary_pos=sp)

    torch.cuda.synchronize()
    time.sleep(idle)
    wall, dev_ms = time_region(step, steps, warmup)
    kern_ms = dev_ms / steps
    return {
        "workload": name, "chunks": chunks, "seqlen_q": Sq, "q_heads": Hq, "kv_heads": Hkv, "head_dim": D,
        "sliding_chunk_num": W, "non_empty_tiles_128x64": tiles, "non_empty_block_tflop": flops / 1e12,
        "steps": steps, "ms_per_step": wall * 1e3 / steps,
        "roofline": {"bound": "mfma", "achieved": flops / (kern_ms * 1e-3) / 1e12, "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": flops / (kern_ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
                     "traffic": None, "kernel": "ksa_prefill_kernel<bf16,128>", "kernel_ms": kern_ms},
    }


def cpu_baseline_prefill(chunks, Hq, Hkv, D, C, S, W, tiles_per_mtile, budget_s=20.0):
    """The reference's CPU path (block mode, restated in oracle/cpu_path.py) on a bounded
    sample of 4096-row query blocks; rate in the same non-empty-block TFLOP/s unit."""
    import torch
    from oracle import cpu_path
    Sq = chunks * (C + S)
    torch.manual_seed(0)
    scale = D ** -0.5
    k = (torch.randn(Sq, Hkv, D) * scale).bfloat16().float()
    v = (torch.randn(Sq, Hkv, D) * scale).bfloat16().float()
    nblk = -(-Sq // cpu_path.BLOCK_ROWS)
    pick = sorted({0, nblk // 4, nblk // 2, (3 * nblk) // 4, nblk - 1})
    # non-empty 128 x 64 tiles of the sampled rows come from the (parity-checked) block index
    done_tiles, t_used, blocks = 0, 0.0, []
    for bi in pick:
        q0 = bi * cpu_path.BLOCK_ROWS
        q1 = min(Sq, q0 + cpu_path.BLOCK_ROWS)
        q = (torch.randn(q1 - q0, Hq, D) * scale).bfloat16().float()
        t0 = time.perf_counter()
        cpu_path.block_mode_rows(q, k, v, q0, C, S, W)
        dt = time.perf_counter() - t0
        tiles = int(tiles_per_mtile[q0 // 128:-(-q1 // 128)].sum())
        done_tiles += tiles
        t_used += dt
        blocks.append(bi)
        if t_used > budget_s:
            break
    flops = 4.0 * 128 * 64 * D * Hq * done_tiles
    return {
        "value": flops / t_used / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"query blocks {blocks} of {nblk} (4096 rows each) of the same workload, "
                  f"fp32 torch SDPA block mode with KV expanded to {Hq} heads, {t_used:.1f} s",
    }


def cpu_baseline_decode(Hq, Hkv, D, rows, nseq=4):
    import torch
    from oracle import cpu_path
    torch.manual_seed(0)
    q = torch.randn(nseq, Hq, 1, D)
    k = torch.randn(nseq, Hkv, rows, D)
    v = torch.randn(nseq, Hkv, rows, D)
    cpu_path.decode_sdpa(q, k, v, Hq // Hkv)
    t0 = time.perf_counter()
    reps = 5
    for _ in range(reps):
        cpu_path.decode_sdpa(q, k, v, Hq // Hkv)
    dt = (time.perf_counter() - t0) / reps
    return {"us_per_sequence": dt / nseq * 1e6, "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{nseq} of 64 sequences, {rows} rows, repeat_kv + fp32 torch SDPA"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--prefill-chunks", type=int, default=1024, help="1024 = 128k text tokens (cfg 2)")
    ap.add_argument("--sliding-chunk-num", type=int, default=4)
    ap.add_argument("--decode-batch", type=int, default=64)
    ap.add_argument("--decode-splits", type=int, default=0, help="0 = library heuristic")
    ap.add_argument("--idle", type=float, default=1.0, metavar="SECONDS",
                    help="idle time before each timed section, so that every section starts from the "
                         "same (idle) power state instead of the one its predecessor left")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--skip-decode", action="store_true")
    ap.add_argument("--skip-prefill", action="store_true")
    ap.add_argument("--skip-pre-attention", action="store_true",
                    help="do not time the fused pre-attention step (q/k RMSNorm + rotary + layout write "
                         "at the prefill shape, reported under 'pre_attention')")
    ap.add_argument("--sustain", type=float, default=3.0, metavar="SECONDS",
                    help="also loop the prefill launch for SECONDS and report the rate of the second "
                         "half under 'sustained' (the chip lowers its clock under a long MFMA load); 0 = skip")
    ap.add_argument("--skip-small-prefill", action="store_true",
                    help="do not time the two smaller prefill configurations (cfg 0: 32 chunks, 16/8 heads; "
                         "cfg 1: 256 chunks, 32/8 heads), reported under 'prefill_cfg0' / 'prefill_cfg1'")
    ap.add_argument("--no-e2e", action="store_true",
                    help="skip the end-to-end decoder (random-init 4B shape: 36 layers, 3 Summary : 1 "
                         "full, batch 8, 32k-token prompt, 256 greedy steps; prefill and decode tokens/s "
                         "under 'e2e')")
    ap.add_argument("--e2e-eager", action="store_true",
                    help="launch the decode steps of the end-to-end run one kernel at a time instead of "
                         "replaying the non-boundary steps from a HIP graph")
    ap.add_argument("--e2e-batch", type=int, default=8)
    ap.add_argument("--e2e-prompt", type=int, default=32768)
    ap.add_argument("--e2e-new", type=int, default=256)
    ap.add_argument("--e2e-layers", type=int, default=36)
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one ksa_copy_rows of 1 GiB (a plain copy kernel of known size, "
                         "used to scale the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    args = ap.parse_args()
    args.e2e = not args.no_e2e
    args.e2e_graph = not args.e2e_eager
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (both kernels shard "
              "by head / sequence with no communication); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    import ksa_amd
    from ksa_amd import _lib

    assert torch.cuda.is_available(), "bench.py needs an MI355X"
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    C, S, D, Hq, Hkv = 128, 8, 128, 32, 8
    W = args.sliding_chunk_num
    result = {
        "metric": "prefill non-empty-block TFLOP/s @128k; decode step us + HBM GB/s (bs=64)",
        "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic (seed 0; q,k,v ~ N(0,1)/sqrt(128) for prefill, N(0,1) for decode)",
        "device": torch.cuda.get_device_name(0), "cu_count": _lib.lib().ksa_device_cu_count(),
        "idle_before_each_section_s": args.idle,
    }

    if args.calibrate_copy:
        from ksa_amd.cache import _move_rows
        rows = 2 ** 30 // (8 * 128 * 2)          # 1 GiB = rows x 8 heads x 128 dims x 2 B
        src = torch.ones(1, 8, rows, 128, dtype=torch.bfloat16, device=dev)
        dst = torch.empty_like(src)
        _move_rows(src, dst, rows)
        torch.cuda.synchronize()
        result["calibration_copy_bytes"] = rows * 8 * 128 * 2
        del src, dst

    # ------------------------------------------------------------------ prefill
    if not args.skip_prefill:
        chunks = args.prefill_chunks
        Sq = chunks * (C + S)
        P = chunks * S
        q, k, v, sp = prefill_inputs(chunks, Hq, Hkv, D, C, S, dev, seed=0)
        idx = ksa_amd.compute_block_sparsity(Sq, Sq + P, C, S, W)
        tiles_per_mtile = (idx[0] + idx[2]).flatten().cpu().numpy()
        tiles = int(tiles_per_mtile.sum())
        flops = 4.0 * 128 * 64 * D * Hq * tiles
        t_idx0 = time.perf_counter()
        ksa_amd.compute_block_sparsity(Sq, Sq + P, C, S, W)
        torch.cuda.synchronize()
        idx_ms = (time.perf_counter() - t_idx0) * 1e3

        def step():
            ksa_amd.summary_attn_func(q, k, v, C, S, W, summary_pos=sp)

        torch.cuda.synchronize()
        time.sleep(args.idle)
        wall, dev_ms = time_region(step, args.steps, args.warmup)
        ms = wall * 1e3 / args.steps
        kern_ms = dev_ms / args.steps
        result.update({
            "value": flops / (wall / args.steps) / 1e12,
            "ms_per_step": ms,
            "config": {"workload": f"cfg2-prefill-128k" if chunks == 1024 else f"prefill-{chunks}-chunks",
                       "chunks": chunks, "seqlen_q": Sq, "prefix_summaries": P, "q_heads": Hq,
                       "kv_heads": Hkv, "head_dim": D, "chunk_size": C, "summary_num": S,
                       "sliding_chunk_num": W, "non_empty_tiles_128x64": tiles,
                       "non_empty_block_tflop": flops / 1e12, "block_index_ms": idx_ms},
            "roofline": {"bound": "mfma", "achieved": flops / (kern_ms * 1e-3) / 1e12,
                         "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                         "frac": flops / (kern_ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
                         "traffic": None, "kernel": "ksa_prefill_kernel<bf16,128>",
                         "kernel_ms": kern_ms},
        })
        if args.sustain > 0:
            rate, clk = sustained_rate(step, flops, args.sustain, 10)
            result["sustained"] = {"seconds": args.sustain, "tflops_second_half": rate,
                                   "frac_of_peak": rate / PEAK_BF16_TFLOPS, "sclk_mhz_mean": clk}
        del q, k, v, sp
        torch.cuda.empty_cache()
        if not args.skip_small_prefill and chunks == 1024:
            # the two smaller configurations of the same kernel (launches of 30 us and 1 ms:
            # more of them per region)
            result["prefill_cfg0"] = prefill_record("cfg0-prefill-32-chunks-16q8kv", 32, 16, 8, D, C, S, W, dev,
                                                    args.steps * 20, args.warmup * 4, args.idle)
            result["prefill_cfg1"] = prefill_record("cfg1-prefill-32k", 256, Hq, Hkv, D, C, S, W, dev,
                                                    args.steps * 4, args.warmup * 2, args.idle)

    # ------------------------------------------------------------------ decode
    if not args.skip_decode:
        torch.cuda.synchronize()
        time.sleep(args.idle)
        Bz = args.decode_batch
        n_chunks_done = 1024
        ws = W * C
        n_sum = n_chunks_done * S
        cap = S + C + ws + n_sum + max(512, n_sum + 256)
        g = torch.Generator(device=dev).manual_seed(1)
        kc = torch.empty(Bz, Hkv, cap, D, dtype=torch.bfloat16, device=dev)
        vc = torch.empty_like(kc)
        for b in range(Bz):
            kc[b] = torch.randn(Hkv, cap, D, generator=g, device=dev).to(torch.bfloat16)
            vc[b] = torch.randn(Hkv, cap, D, generator=g, device=dev).to(torch.bfloat16)
        qd = torch.randn(Bz, Hq, 1, D, generator=g, device=dev).to(torch.bfloat16)
        cbl = torch.randint(0, C, (Bz,), generator=g, device=dev, dtype=torch.int32) + 1  # after update_text
        start = (S + C - cbl).to(torch.int32)
        end = torch.full((Bz,), S + C + ws + n_sum - min(W * S, n_sum), dtype=torch.int32, device=dev)
        L = (end - start).to(torch.int64)
        bytes_step = int((2 * L * Hkv * D * 2 + 2 * Hq * D * 2).sum())
        nsplit = args.decode_splits or _lib.lib().ksa_decode_auto_splits(Bz, Hkv, cap)

        def dstep():
            ksa_amd.ksa_decode(qd, kc, vc, start, end, nsplit=nsplit)

        wall, dev_ms = time_region(dstep, args.steps, args.warmup)
        us = dev_ms * 1e3 / args.steps
        result["decode"] = {
            "workload": "cfg3-decode-bs64-128k" if Bz == 64 else f"decode-bs{Bz}",
            "batch": Bz, "rows_per_sequence_mean": float(L.float().mean()), "cache_rows": cap,
            "nsplit": nsplit, "us_per_step": us, "us_per_step_wall": wall * 1e6 / args.steps,
            "algorithmic_bytes": bytes_step, "hbm_gbps": bytes_step / (us * 1e-6) / 1e9,
            "roofline": {"bound": "hbm", "achieved": bytes_step / (us * 1e-6) / 1e9,
                         "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                         "frac": bytes_step / (us * 1e-6) / 1e9 / PEAK_HBM_GBPS, "traffic": None,
                         "kernel": "ksa_decode_kernel<bf16,128> (+ merge when nsplit > 1)"},
        }
        if args.skip_prefill:
            result.update({"value": result["decode"]["hbm_gbps"], "unit": "GB/s",
                           "ms_per_step": us / 1e3,
                           "config": {"workload": result["decode"]["workload"]},
                           "roofline": result["decode"]["roofline"]})
        del kc, vc
        torch.cuda.empty_cache()

    # ------------------------------------------------------------------ pre-attention step
    if not args.skip_pre_attention:
        torch.cuda.synchronize()
        time.sleep(args.idle)
        chunks = args.prefill_chunks
        Sp = chunks * (C + S)
        g = torch.Generator(device=dev).manual_seed(2)
        qkv = torch.randn(1, Sp, (Hq + 2 * Hkv) * D, generator=g, device=dev).to(torch.bfloat16)
        qp = qkv[..., : Hq * D].view(1, Sp, Hq, D)
        kp = qkv[..., Hq * D: (Hq + Hkv) * D].view(1, Sp, Hkv, D)
        vp = qkv[..., (Hq + Hkv) * D:].view(1, Sp, Hkv, D)
        wq = torch.ones(D, dtype=torch.bfloat16, device=dev)
        ang = torch.arange(Sp, device=dev, dtype=torch.float32)[:, None] * \
            (1.0 / 10000.0 ** (torch.arange(0, D, 2, device=dev, dtype=torch.float32) / D))[None]
        emb = torch.cat((ang, ang), dim=-1)
        cosb, sinb = emb.cos().to(torch.bfloat16)[None], emb.sin().to(torch.bfloat16)[None]
        qo, ko, vo = torch.empty_like(qp), torch.empty_like(kp), torch.empty_like(vp)

        def pstep():
            ksa_amd.pre_attention(qp, kp, vp, wq, wq, cosb, sinb, 1e-6, q_out=qo, k_out=ko, v_out=vo)

        wall, dev_ms = time_region(pstep, args.steps, args.warmup)
        us = dev_ms * 1e3 / args.steps
        pbytes = 2 * Sp * (Hq + 2 * Hkv) * D * 2 + 2 * Sp * D * 2   # q, k, v in and out; cos, sin in
        result["pre_attention"] = {
            "workload": f"pre-attention-{chunks}-chunks-{Hq}q{Hkv}kv",
            "what": "q/k RMSNorm on head_dim + rotary embedding + write of q, k, v in the attention layout",
            "us_per_step": us, "algorithmic_bytes": pbytes, "hbm_gbps": pbytes / (us * 1e-6) / 1e9,
            "roofline": {"bound": "hbm", "achieved": pbytes / (us * 1e-6) / 1e9, "peak": PEAK_HBM_GBPS,
                         "unit": "GB/s", "frac": pbytes / (us * 1e-6) / 1e9 / PEAK_HBM_GBPS, "traffic": None,
                         "kernel": "ksa_pre_attention_kernel<bf16,128>"},
        }
        del qkv, qo, ko, vo, cosb, sinb, emb, ang
        torch.cuda.empty_cache()

    # ------------------------------------------------------------------ end-to-end decoder (config 4)
    if args.e2e:
        from ksa_amd.model import KsaQwen3Config, KsaQwen3ForCausalLM, init_weights
        nl = args.e2e_layers
        cfg = KsaQwen3Config(num_hidden_layers=nl,
                             summary_sliding_chunk_num=[(1 << 20) if i % 4 == 3 else W for i in range(nl)])
        weights = init_weights(cfg, dev, torch.bfloat16, seed=0)
        model = KsaQwen3ForCausalLM(cfg, weights)
        gi = torch.Generator(device=dev).manual_seed(3)
        ids = torch.randint(0, cfg.vocab_size, (args.e2e_batch, args.e2e_prompt), generator=gi, device=dev)
        # library set-up (GEMM handles, index cache, every kernel of the decode path loaded once)
        model.generate(ids[:, :300], 4, use_graph=bool(args.e2e_graph))
        torch.cuda.synchronize()
        # the cache hand-off inside the prefill, timed with events on the launch stream
        reorg_ev = []
        cache_cls = model.ops.cache_cls

        class TimedCache(cache_cls):   # (the prefill reorganises a layer's rows as soon as its attention has run)
            def reorganize_layer(self, layer, summary_mask):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                super().reorganize_layer(layer, summary_mask)
                e1.record()
                reorg_ev.append((e0, e1))
        model.ops.cache_cls = TimedCache
        t0 = time.perf_counter()
        logits, cache = model.prefill(ids)
        torch.cuda.synchronize()
        t_prefill = time.perf_counter() - t0
        model.ops.cache_cls = cache_cls
        reorganize_ms = sum(a.elapsed_time(b) for a, b in reorg_ev)

        # Untimed check of what is about to be timed: eight steps launched eagerly and the same eight
        # replayed from the graph, each on a copy of the cache as the prefill left it, teacher-forced
        # with the eager run's tokens; the logits must agree within 1 % of the logit scale.
        import copy
        n_chk = 8 if args.e2e_graph else 0
        chk_err = None
        if n_chk:
            first = logits.clone()
            c_e = copy.deepcopy(cache)
            toks, ref, lg = [], [], first
            for _ in range(n_chk):
                toks.append(model.ops.argmax(lg[:, 0])[:, None])
                lg = model.decode_step(toks[-1], c_e)
                ref.append(lg[:, 0].float())
            del c_e
            c_g = copy.deepcopy(cache)
            chk_err = 0.0
            for t in range(n_chk):
                lg = model.decode_step_graph(toks[t], c_g)
                scale_ = ref[t].abs().max().item()
                chk_err = max(chk_err, (lg[:, 0].float() - ref[t]).abs().max().item() / scale_)
            del c_g, ref, toks, lg
            torch.cuda.empty_cache()
            assert chk_err <= 1e-2, f"graph decode differs from eager decode by {chk_err} of the logit scale"
            logits = first

        def attended_rows():   # cache rows one decode step reads, summed over the layers
            return sum(e - a for a, e in (cache.attention_range(li) for li in range(nl)))

        def matrix_bytes():    # weights one decode step reads: every layer's matrices and the output head
            n = sum(w.numel() for lw in weights["layers"] for w in lw.values())
            return (n + model.lm_head.numel() + weights["norm"].numel()) * 2

        rows_first = attended_rows()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        n_boundary = 0
        b_ev = []
        for _ in range(args.e2e_new):
            nxt = model.ops.argmax(logits[:, 0])[:, None]
            is_b = cache.get_cur_chunk_size() == cfg.summary_chunk_size - 1
            n_boundary += is_b
            if is_b:
                b_ev.append((torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)))
                b_ev[-1][0].record()
            logits = model.decode_step_graph(nxt, cache) if args.e2e_graph else model.decode_step(nxt, cache)
            if is_b:
                b_ev[-1][1].record()
        torch.cuda.synchronize()
        t_decode = time.perf_counter() - t0
        # pass / fail of the timed run (outside the timed region): no launch gave up waiting, the
        # last logits are finite, the cache counted every token
        model.check_steps(cache)
        assert bool(torch.isfinite(logits.float()).all()), "non-finite logits at the end of the decode run"
        assert cache.get_true_token_num() == args.e2e_prompt + args.e2e_new
        rows_mean = (rows_first + attended_rows()) / 2
        step_bytes = matrix_bytes() + 2 * rows_mean * cfg.num_key_value_heads * cfg.head_dim * 2 * args.e2e_batch
        floor_ms = step_bytes / (PEAK_HBM_GBPS * 1e9) * 1e3
        b_ms = [a.elapsed_time(b) for a, b in b_ev]
        t_in_chunk = t_decode * 1e3 - sum(b_ms)
        result["e2e"] = {
            "workload": f"random-init decoder, {nl} layers (3 Summary W={W} : 1 unbounded window), hidden "
                        f"{cfg.hidden_size}, {Hq}/{Hkv} heads, batch {args.e2e_batch}, prompt "
                        f"{args.e2e_prompt}, {args.e2e_new} greedy steps",
            "checked": True,
            "check": {"graph_vs_eager_steps": n_chk, "graph_vs_eager_max_rel_logit_diff": chk_err,
                      "logits_finite": True, "mlp_one_launch_timeouts": 0},
            "prefill_s": t_prefill, "prefill_tokens_per_s": args.e2e_batch * args.e2e_prompt / t_prefill,
            "reorganize_ms": reorganize_ms,
            "decode_s": t_decode, "decode_ms_per_step": t_decode / args.e2e_new * 1e3,
            "decode_tokens_per_s": args.e2e_batch * args.e2e_new / t_decode,
            "chunk_boundary_steps": int(n_boundary), "boundary_step_ms": (sum(b_ms) / len(b_ms)) if b_ms else None,
            "in_chunk_step_ms": t_in_chunk / max(1, args.e2e_new - len(b_ms)),
            "decode_hip_graph": bool(args.e2e_graph),
            "decode_step_bytes": int(step_bytes), "decode_hbm_floor_ms": floor_ms,
            "decode_frac_of_hbm_floor": floor_ms / (t_decode / args.e2e_new * 1e3),
            "hbm_allocated_gb": torch.cuda.max_memory_allocated() / 1e9,
        }
        del model, weights, cache, logits
        torch.cuda.empty_cache()

    if not args.no_cpu_baseline:
        try:
            Sq_ = args.prefill_chunks * (C + S)
            ix = ksa_amd.compute_block_sparsity(Sq_, Sq_ + args.prefill_chunks * S, C, S, W)
            cb = cpu_baseline_prefill(args.prefill_chunks, Hq, Hkv, D, C, S, W,
                                      (ix[0] + ix[2]).flatten().cpu().numpy())
            if not args.skip_decode:
                cb["decode"] = cpu_baseline_decode(Hq, Hkv, D, 8672 + 64)
            result["cpu_baseline"] = cb
        except Exception as e:  # the baseline is a reported extra, never the measured path
            result["cpu_baseline"] = {"error": repr(e)}

    # HBM traffic per launch comes from a separate rocprofv3 --pmc measurement (FETCH_SIZE and
    # WRITE_SIZE, scaled by a copy kernel of known size); the summary is kept under profiles/
    tfile = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    if os.path.exists(tfile):
        try:
            t = json.load(open(tfile))
            if "roofline" in result and result.get("config", {}).get("workload") == t.get("prefill_workload"):
                result["roofline"]["traffic"] = t.get("prefill_bytes_per_launch")
            if "decode" in result and result["decode"]["workload"] == t.get("decode_workload"):
                result["decode"]["roofline"]["traffic"] = t.get("decode_bytes_per_launch")
            if "pre_attention" in result and t.get("pre_attention_workload") == result["pre_attention"]["workload"]:
                result["pre_attention"]["roofline"]["traffic"] = t.get("pre_attention_bytes_per_launch")
            for key in ("prefill_cfg0", "prefill_cfg1"):
                if key in result and result[key]["workload"] == t.get(key + "_workload"):
                    result[key]["roofline"]["traffic"] = t.get(key + "_bytes_per_launch")
        except Exception:
            pass
    _mark_traffic_source(result)
    print(json.dumps(result))


def _mark_traffic_source(result):
    """Every `roofline.traffic` that is set gets its provenance next to it: these are not read in this
    run but taken from a separate counter run whose summary is committed."""
    src = "profiles/hbm_traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, separate run on another box)"
    recs = [result] + [result[k] for k in ("decode", "pre_attention", "prefill_cfg0", "prefill_cfg1") if k in result]
    for r in recs:
        rf = r.get("roofline")
        if rf is not None and rf.get("traffic") is not None:
            rf["traffic_source"] = src


if __name__ == "__main__":
    main()

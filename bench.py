#!/usr/bin/env python3
"""Benchmark of the MI355X paged-attention hot path (one GPU).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--configs 1,2,3,4,5] [--no-check]

A step is one pass of the hot path over one batch of synthetic input that is already
resident in HBM: the decode operator for the decode shapes, KV-store + extend attention
for the chunked-prefill shape, the prefill operator for the speculative-verify shape.
Every step is bracketed by HIP events on the stream the kernels are launched on; the
median, minimum and mean over the timed steps are reported.

The last line of stdout is ONE JSON object.  Its headline (`value`) is decode-attention
HBM throughput on shape 2 (Qwen3-8B-shaped paged decode, batch 64); `prefill` carries
the chunked-prefill TFLOP/s of shape 3 and `all_configs` one row per benchmark shape.
`roofline.achieved` is ALGORITHMIC bytes (or flops) per step divided by the mean step
time, which includes the small LSE-merge launch that follows the attention kernel.
`cpu_baseline` times the CPU oracle (float build, OpenMP) on a bounded sample of the same
workload on this machine's host cores: a reported baseline, not a target.
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "mini-sglang-mlx_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

METRIC = "decode attn HBM TB/s (% of peak) + chunked-prefill attn TFLOP/s (% MFMA peak)"
HBM_PEAK = 8.0e12
MFMA_PEAK = 2.5e15
INFINITY_CACHE_BYTES = 256e6  # MI355X memory-side cache
SPINUP_MS = 100.0  # untimed run of the step before its warm-up steps (clock settling)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def time_steps(fn, steps: int, warmup: int, spinup_ms: float = SPINUP_MS):
    """`warmup` untimed steps, then exactly `steps` back-to-back steps between two HIP events
    recorded on torch's current stream (the stream every operator launches on), bracketed by
    device syncs: that mean is the reported figure.  Two diagnostic passes follow: one that
    brackets every step with its own event pair (min / median / the per-step list; those carry
    the event markers' own few microseconds), and a repeat of the first pass, which shows
    whether the first one still saw the clocks settling."""
    import torch

    probe = _ClockProbe()

    def loop_ms():
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        probe.arm()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0.record()
        try:
            for _ in range(steps):
                fn()
        finally:
            probe.disarm()
        e1.record()
        torch.cuda.synchronize()
        time_steps.last_shader_ghz = probe.ghz()
        return e0.elapsed_time(e1), (time.perf_counter() - t0) * 1e3

    # The shader clock needs some tens of milliseconds of load to settle (measured: the MFMA
    # kernels keep getting faster for the first ~30 ms after an idle spell), so the step first
    # runs untimed for SPINUP_MS of device time; the `warmup` steps the caller asked for follow.
    spin0 = torch.cuda.Event(enable_timing=True)
    spin0.record()
    while True:
        for _ in range(4):
            fn()
        spin1 = torch.cuda.Event(enable_timing=True)
        spin1.record()
        spin1.synchronize()
        if spin0.elapsed_time(spin1) >= spinup_ms:
            break
    for _ in range(warmup):
        fn()
    loop, wall_ms = loop_ms()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    for i in range(steps):
        starts[i].record()
        fn()
        ends[i].record()
    torch.cuda.synchronize()
    per = [s.elapsed_time(e) for s, e in zip(starts, ends)]
    ghz = time_steps.last_shader_ghz  # of the reported pass
    again, _ = loop_ms()
    time_steps.last_repeat_ms = again / steps
    time_steps.last_shader_ghz = ghz
    return loop / steps, per, wall_ms


class _ClockProbe:
    """Shader clock under the attention kernels of a timed loop: the library's measurement aid
    (MSGL_TUNE_CLOCK_PROBE) makes workgroup 0 of every attention kernel leave the shader cycles
    and the 100 MHz wall ticks it lived for in two device words; read after the loop, they are
    those of its last launch."""

    def __init__(self):
        import torch

        from mini_sglang_amd_kernel import _lib

        self._lib = _lib
        self.buf = torch.zeros(2, dtype=torch.int64, device="cuda")

    def arm(self):
        self.buf.zero_()
        self._lib.set_tuning(self._lib.TUNE_CLOCK_PROBE, self.buf.data_ptr())

    def disarm(self):
        self._lib.set_tuning(self._lib.TUNE_CLOCK_PROBE, 0)

    def ghz(self):
        cycles, ticks = self.buf.tolist()
        return cycles / ticks * 0.1 if ticks > 0 else None


def make_step(g):
    from mini_sglang_amd_kernel import (paged_decode_attention, paged_prefill_attention,
                                        store_kv_cache)

    if g.kind == "decode":
        def step():
            return paged_decode_attention(g.q, g.k_cache, g.v_cache, g.kv_indptr, g.kv_indices,
                                          g.num_kv_splits, g.sm_scale, g.max_kv_splits)
    else:
        def step():
            if g.out_loc is not None:
                store_kv_cache(g.k_cache, g.v_cache, g.out_loc, g.new_k, g.new_v)
            return paged_prefill_attention(
                g.q, g.k_cache, g.v_cache, g.qo_indptr, g.kv_indptr, g.kv_indices,
                g.prefix_lens, g.sm_scale, g.max_len_extend,
                is_cross_attention=g.is_cross_attention,
                sliding_window_size=g.sliding_window_size)
    return step


def oracle_run(c, precision):
    import oracle

    if c.out_loc is not None:
        c = c.clone_pools()
        oracle.store_kv_cache(c.k_cache, c.v_cache, c.out_loc, c.new_k, c.new_v)
    if c.kind == "decode":
        return oracle.paged_decode_attention(
            c.q, c.k_cache, c.v_cache, c.kv_indptr, c.kv_indices, c.num_kv_splits, c.sm_scale,
            c.max_kv_splits, precision=precision, return_f32=True)[1], c
    return oracle.paged_prefill_attention(
        c.q, c.k_cache, c.v_cache, c.qo_indptr, c.kv_indptr, c.kv_indices, c.prefix_lens,
        c.sm_scale, c.max_len_extend, is_cross_attention=c.is_cross_attention,
        sliding_window_size=c.sliding_window_size, precision=precision, return_f32=True)[1], c


def sample_requests(wl, max_flops: float):
    """Requests, shortest first, whose oracle cost stays within ``max_flops`` (at least one)."""
    from mini_sglang_amd import roofline

    cost = []
    for b in range(wl.batch):
        p = wl.kv_lens[b] - wl.extend_lens[b]
        cost.append((4 * wl.head_dim * wl.n_q * roofline.visible_pairs(
            p, wl.extend_lens[b], wl.kv_lens[b], wl.is_cross_attention,
            wl.sliding_window_size), b))
    cost.sort()
    picked, total = [], 0.0
    for c, b in cost:
        if picked and total + c > max_flops:
            break
        picked.append(b)
        total += c
    return sorted(picked), total


def run_config(cfg: int, variant: str, steps: int, warmup: int, check: bool, cpu_budget_flops: float,
               dev):
    import torch

    from mini_sglang_amd.workloads import config_workload

    t0 = time.time()
    # multi-GiB pools of the long-context shape are drawn on the GPU; the rest on the host
    if variant == "head_dim_256":
        wl = config_workload(cfg, head_dim=256)
    else:
        wl = config_workload(cfg, variant=variant, pool_device=dev if cfg == 4 else None)
    g = wl.to(dev)
    gen_s = time.time() - t0
    step = make_step(g)
    out = step()
    torch.cuda.synchronize()
    mean_ms, per, wall_ms = time_steps(step, steps, warmup)
    med_ms = statistics.median(per)
    abytes = wl.attention_bytes()
    aflops = wl.attention_flops()
    sbytes = wl.store_bytes()
    bound = "mfma" if (wl.kind == "prefill" and wl.max_len_extend * (wl.n_q // wl.n_kv) > 64) else "hbm"
    row = {
        "config": cfg, "workload": wl.name, "kind": wl.kind, "batch": wl.batch,
        "n_q": wl.n_q, "n_kv": wl.n_kv, "head_dim": wl.head_dim, "page_size": wl.page_size,
        "total_kv_tokens": int(sum(wl.kv_lens)), "total_q_tokens": int(sum(wl.extend_lens)),
        "sliding_window": wl.sliding_window_size,
        "ms_mean": mean_ms, "ms_median": med_ms, "ms_min": min(per),
        "ms_mean_repeat": time_steps.last_repeat_ms, "spinup_ms": SPINUP_MS,
        # shader clock under the attention kernel of the last timed step (None: no such kernel ran)
        "shader_ghz": time_steps.last_shader_ghz,
        "per_step_us": [round(x * 1e3, 1) for x in per],
        "wall_ms_per_step": wall_ms / steps, "steps": steps, "warmup": warmup,
        "algorithmic_bytes": abytes, "algorithmic_flops": aflops, "store_bytes": sbytes,
        "bound": bound, "gen_s": round(gen_s, 1),
    }
    if bound == "hbm":
        row["achieved_TBps"] = abytes / (mean_ms * 1e-3) / 1e12
        row["roofline_frac"] = row["achieved_TBps"] * 1e12 / HBM_PEAK
        row["cache_resident"] = abytes < INFINITY_CACHE_BYTES  # fits the Infinity Cache: latency-bound
    else:
        row["achieved_TFLOPs"] = aflops / (mean_ms * 1e-3) / 1e12
        row["roofline_frac"] = row["achieved_TFLOPs"] * 1e12 / MFMA_PEAK

    if check or cpu_budget_flops > 0:
        import oracle  # noqa: F401  (checker and CPU baseline only)

        reqs, flops = sample_requests(wl, max(cpu_budget_flops, 2e10))
        sub = wl.select(reqs).to("cpu")
        torch.set_num_threads(os.cpu_count() or 1)
        # untimed pass over the shortest request: loads the oracle library, starts the OpenMP team
        oracle_run(wl.select(reqs[:1]).to("cpu"), "f32")
        t1 = time.perf_counter()
        want, ref = oracle_run(sub, "f32")
        cpu_s = time.perf_counter() - t1
        if check:
            gsub = sub.to(dev)
            got = make_step(gsub)()
            torch.cuda.synchronize()
            diff = (got.float().cpu() - want).abs()
            row["max_abs_err"] = float(diff.max())
            row["mean_abs_err"] = float(diff.mean())
            row["checked_requests"] = len(reqs)
            row["parity_ok"] = bool(row["max_abs_err"] <= 2e-2 and row["mean_abs_err"] <= 2e-3)
            if sub.out_loc is not None:
                row["kv_pool_bit_exact"] = bool(
                    torch.equal(gsub.k_cache.cpu().view(torch.int16), ref.k_cache.view(torch.int16))
                    and torch.equal(gsub.v_cache.cpu().view(torch.int16), ref.v_cache.view(torch.int16)))
        threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
        cpu = {"seconds": cpu_s, "cores": threads, "kind": "port",
               "sample": f"{len(reqs)} of {wl.batch} requests (shortest first), CPU oracle float "
                         f"build with OpenMP, one timed pass after a warm-up pass on one request, "
                         f"MLX not installed"}
        if bound == "hbm":
            cpu["value"] = sub.attention_bytes() / cpu_s / 1e12
            cpu["unit"] = "TB/s"
        else:
            cpu["value"] = sub.attention_flops() / cpu_s / 1e12
            cpu["unit"] = "TFLOP/s"
        row["cpu_baseline"] = cpu
    del g, out
    torch.cuda.empty_cache()
    return row


def load_traffic():
    """Measured HBM bytes per launch (rocprofv3 FETCH_SIZE + WRITE_SIZE, calibrated against a
    copy of known size) for the workloads that have a committed counter summary."""
    path = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    if os.path.exists(path):
        with open(path) as f:
            return {k: v.get("total_bytes") for k, v in json.load(f).items()}
    return {}


def run_metadata_build(dev, steps: int, warmup: int, cpu_baseline: bool):
    """On-device build of a step's CSR metadata from the slot table, at the sizes of shape 2
    (64 requests, ~295 K kv tokens) and shape 4 (16 requests, ~1.3 M kv tokens).  Integer copy
    work: 8 bytes per kv token (slot id read + written) plus 4 per request array entry."""
    import numpy as np
    import torch

    from mini_sglang_amd_kernel import build_attention_metadata

    rows_out = []
    for name, batch, lo, hi in (("shape2_sizes", 64, 1024, 8192), ("shape4_sizes", 16, 32768, 131072)):
        g = torch.Generator().manual_seed(0x5EED0100 + batch)
        kv = torch.randint(lo, hi + 1, (batch,), generator=g, dtype=torch.int32)
        table = torch.randint(0, 2 ** 31 - 1, (batch + 1, hi), generator=g, dtype=torch.int32)
        trows = torch.randperm(batch, generator=g).to(torch.int32)
        total = int(kv.sum())
        d_table, d_rows, d_kv = table.to(dev), trows.to(dev), kv.to(dev)

        def step():
            return build_attention_metadata(d_table, d_rows, d_kv, None, total_kv=total)

        out = step()
        torch.cuda.synchronize()
        mean_ms, per, _ = time_steps(step, steps, warmup)
        abytes = 8 * total + 4 * (5 * batch + 2)
        row = {"sizes": name, "batch": batch, "total_kv_tokens": total, "us_mean": mean_ms * 1e3,
               "us_min": min(per) * 1e3, "algorithmic_bytes": abytes,
               "achieved_GBps": abytes / (mean_ms * 1e-3) / 1e9,
               "cache_resident": abytes < 2 * INFINITY_CACHE_BYTES, "launch_bound": mean_ms * 1e3 < 25.0}
        if cpu_baseline:
            from oracle import metadata_oracle  # checker and CPU baseline only

            t1 = time.perf_counter()
            want = metadata_oracle.build_decode_metadata(table.numpy(), trows.numpy(), kv.numpy())
            cpu_s = time.perf_counter() - t1
            row["cpu_port_us"] = cpu_s * 1e6
            row["exact"] = bool(np.array_equal(out["kv_indices"].cpu().numpy(), want["kv_indices"])
                                and np.array_equal(out["kv_indptr"].cpu().numpy(), want["kv_indptr"])
                                and np.array_equal(out["num_kv_splits"].cpu().numpy(),
                                                   want["num_kv_splits"]))
        log(f"[metadata] {name}: {row['us_mean']:.1f} us mean ({row['us_min']:.1f} min)  "
            f"{row['achieved_GBps']:.0f} GB/s  cpu {row.get('cpu_port_us', float('nan')):.0f} us  "
            f"exact {row.get('exact')}")
        rows_out.append(row)
    return rows_out


def run_norm_rope_store(dev, steps: int, warmup: int, cpu_baseline: bool):
    """Fused q/k RMSNorm + rotary embedding + KV-store at the token counts of shape 3 (4096 new
    tokens) and shape 2 (64), 32 q / 8 kv heads of 128.  Every element of q, k, v is read once
    and written once: 2 * (n_q + 2 n_kv) * d * 2 bytes per token + 8 (position, slot)."""
    import numpy as np
    import torch

    from mini_sglang_amd_kernel import qk_norm_rope_store

    n_q, n_kv, d = 32, 8, 128
    rows_out = []
    for name, L in (("shape3_new_tokens", 4096), ("shape2_new_tokens", 64)):
        g = torch.Generator().manual_seed(0x5EED0200 + L)
        mk = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16)
        q, k, v = mk(L, n_q, d), mk(L, n_kv, d), mk(L, n_kv, d)
        qw, kw = (1 + 0.1 * torch.randn(d, generator=g)).to(torch.bfloat16), (1 + 0.1 * torch.randn(d, generator=g)).to(torch.bfloat16)
        slots = 2 * L + 64
        pos = torch.randint(0, 16384, (L,), generator=g, dtype=torch.int32)
        loc = torch.randperm(slots, generator=g)[:L].to(torch.int32)
        kc, vc = torch.zeros(slots, n_kv, d, dtype=torch.bfloat16), torch.zeros(slots, n_kv, d, dtype=torch.bfloat16)
        dq, dk, dv, dqw, dkw, dpos, dloc, dkc, dvc = (t.to(dev) for t in (q, k, v, qw, kw, pos, loc, kc, vc))

        def step():
            return qk_norm_rope_store(dq, dk, dv, dqw, dkw, dpos, dloc, dkc, dvc, eps=1e-6, rope_base=1e6)

        out = step()
        torch.cuda.synchronize()
        mean_ms, per, _ = time_steps(step, steps, warmup)
        abytes = L * (2 * (n_q + 2 * n_kv) * d * 2 + 8)
        row = {"sizes": name, "tokens": L, "us_mean": mean_ms * 1e3, "us_min": min(per) * 1e3,
               "algorithmic_bytes": abytes, "achieved_GBps": abytes / (mean_ms * 1e-3) / 1e9,
               "hbm_frac": abytes / (mean_ms * 1e-3) / HBM_PEAK,
               # the same buffers every step: what fits twice into the Infinity Cache is a cache
               # figure, not a memory figure; a step under ~25 us is launch and latency
               "cache_resident": abytes < 2 * INFINITY_CACHE_BYTES,
               "launch_bound": mean_ms * 1e3 < 25.0}
        if cpu_baseline:
            from oracle import qk_norm_rope_oracle as qo  # checker and CPU baseline only

            n = min(L, 512)
            f = lambda t: t.float().numpy()
            t1 = time.perf_counter()
            wq, wkc, wvc = qo.qk_norm_rope_store(f(q[:n]), f(k[:n]), f(v[:n]), f(qw), f(kw), pos[:n].numpy(),
                                                 loc[:n].numpy(), f(kc), f(vc), 1e-6, 1e6)
            cpu_s = time.perf_counter() - t1
            row["cpu_port_GBps"] = n * (2 * (n_q + 2 * n_kv) * d * 2 + 8) / cpu_s / 1e9
            row["cpu_sample"] = f"first {n} tokens, numpy port, 1 core"
            dq_err = (out[:n].float().cpu().numpy() - wq)
            row["q_max_abs_err"] = float(np.abs(dq_err).max())
            row["v_rows_bit_exact"] = bool(np.array_equal(dvc.float().cpu().numpy()[loc[:n].numpy()],
                                                          wvc[loc[:n].numpy()]))
        log(f"[norm+rope+store] {name}: {row['us_mean']:.1f} us mean ({row['us_min']:.1f} min)  "
            f"{row['achieved_GBps']:.0f} GB/s ({row['hbm_frac']*100:.1f}% of hbm peak)  "
            f"cpu {row.get('cpu_port_GBps', float('nan')):.3f} GB/s  err {row.get('q_max_abs_err')}")
        rows_out.append(row)
    return rows_out


def run_gdn_state(dev, steps: int, warmup: int, cpu_baseline: bool):
    """Gated delta-rule state kernel at the reference's benchmark sizes (hk 16, hv 32,
    dk = dv = 128; test_and_bench/gdn_state.py:33-48): decode of 8 requests (HBM-bound, the
    fp32 state of every (request, head) read and written once) and a 1024-token prefill (a
    serial chain per state row)."""
    import numpy as np
    import torch

    from mini_sglang_amd_kernel import gdn_state_inplace

    hk, hv, d = 16, 32, 128
    rows_out = []
    for name, lengths, single in (("decode_batch8", [1] * 8, True), ("decode_batch64", [1] * 64, True),
                                  ("prefill_1024", [1024], False)):
        g = torch.Generator().manual_seed(0x5EED0300 + len(lengths))
        T, B = sum(lengths), len(lengths)
        bf = lambda *s: (0.05 * torch.randn(*s, generator=g)).to(torch.bfloat16)
        sg = lambda *s: torch.sigmoid(torch.randn(*s, generator=g)).to(torch.bfloat16)
        q, k, v, gg, beta = bf(T, hk, d), bf(T, hk, d), bf(T, hv, d), sg(T, hv), sg(T, hv)
        state = 0.05 * torch.randn(B + 1, hv, d, d, generator=g)
        slots = torch.arange(B, dtype=torch.int32)
        ip = torch.tensor([0] + list(np.cumsum(lengths)), dtype=torch.int32)
        dq, dk, dv, dg, db, dst, dsl, dip = (t.to(dev) for t in (q, k, v, gg, beta, state, slots, ip))
        state_bytes = 2 * B * hv * d * d * 4
        io_bytes = T * (2 * hk * d * 2 + 2 * hv * d * 2 + 2 * hv * 2)
        # A state pool smaller than twice the 256 MB Infinity Cache would be served from that cache
        # step after step: the steps rotate over as many copies of the pool as it takes to get
        # past it (at most 8), so that the figure is a memory figure.
        pool_bytes = dst.numel() * 4
        copies = max(1, min(8, -(-int(2 * INFINITY_CACHE_BYTES) // max(pool_bytes, 1))))
        pools = [dst] + [dst.clone() for _ in range(copies - 1)]
        turn = [0]

        def step():
            turn[0] = (turn[0] + 1) % copies
            return gdn_state_inplace(dq, dk, dv, dg, db, pools[turn[0]], dsl, dip, single_token_mode=single)

        step()
        torch.cuda.synchronize()
        mean_ms, per, _ = time_steps(step, steps, warmup)
        row = {"sizes": name, "tokens": T, "batch": B, "us_mean": mean_ms * 1e3, "us_min": min(per) * 1e3,
               "algorithmic_bytes": state_bytes + io_bytes,
               "achieved_GBps": (state_bytes + io_bytes) / (mean_ms * 1e-3) / 1e9,
               "tokens_per_s": T / (mean_ms * 1e-3),
               "state_pool_copies_rotated": copies,
               "cache_resident": copies * pool_bytes < 2 * INFINITY_CACHE_BYTES,
               # a step under ~25 us is launch and latency, whatever it moves
               "launch_bound": mean_ms * 1e3 < 25.0}
        if cpu_baseline:
            from oracle import gdn_state_oracle as go  # checker and CPU baseline only

            n = min(T, 8)
            f = lambda t: t.float().numpy()
            nb = B if single else 1
            t1 = time.perf_counter()
            go.gdn_state_inplace(f(q[:n]), f(k[:n]), f(v[:n]), f(gg[:n]), f(beta[:n]), state.numpy(),
                                 slots[:min(nb, n)].numpy(), None if single else np.array([0, n], np.int32),
                                 single_token_mode=single)
            row["cpu_port_tokens_per_s"] = n / (time.perf_counter() - t1)
            row["cpu_sample"] = f"first {n} tokens, numpy float64 port, 1 core"
        log(f"[gdn_state] {name}: {row['us_mean']:.1f} us mean ({row['us_min']:.1f} min)  "
            f"{row['achieved_GBps']:.0f} GB/s  {row['tokens_per_s']:.3g} tokens/s  "
            f"cpu {row.get('cpu_port_tokens_per_s', float('nan')):.3g} tokens/s")
        rows_out.append(row)
    return rows_out


def run_state_pool(dev, steps: int, warmup: int, cpu_baseline: bool):
    """Recurrent-state pool: the batched slot copy that seeds every request's scratch slot from its
    main slot before a replay-style verify, at the gdn benchmark's state size (hv 32, dk = dv = 128
    fp32 = 2 MiB per slot and layer, plus a (3, 8192) bf16 conv state) for 24 layers.  HBM-bound:
    every copied byte is read once and written once."""
    import torch

    from mini_sglang_amd.kvcache import MambaStateConfig, MambaStatePool

    layers, hv, d = 24, 32, 128
    rows_out = []
    for name, batch in (("verify_seed_8_requests", 8), ("verify_seed_32_requests", 32)):
        pool = MambaStatePool(MambaStateConfig(num_slots=2 * batch, num_layers=layers,
                                               conv_shapes=[[(3, 8192)]] * layers,
                                               temporal_shapes=[(hv, d, d)] * layers), device=dev)
        for l in range(layers):
            pool.temporal_state(l).normal_()
        src = torch.arange(1, batch + 1, dtype=torch.int32, device=dev)
        dst = torch.arange(batch + 1, 2 * batch + 1, dtype=torch.int32, device=dev)

        def step():
            pool.copy_batched(src, dst)

        step()
        torch.cuda.synchronize()
        mean_ms, per, _ = time_steps(step, steps, warmup)
        per_slot = layers * (hv * d * d * 4 + 3 * 8192 * 2)
        moved = 2 * batch * per_slot
        exact = all(torch.equal(pool.temporal_state(l)[1:batch + 1], pool.temporal_state(l)[batch + 1:])
                    for l in (0, layers - 1))
        row = {"sizes": name, "pairs": batch, "layers": layers, "us_mean": mean_ms * 1e3,
               "us_min": min(per) * 1e3, "algorithmic_bytes": moved,
               "achieved_GBps": moved / (mean_ms * 1e-3) / 1e9,
               "hbm_frac": moved / (mean_ms * 1e-3) / 8e12, "bit_exact": exact,
               "cache_resident": moved < 2 * INFINITY_CACHE_BYTES, "launch_bound": mean_ms * 1e3 < 25.0}
        if cpu_baseline:
            import numpy as np

            from oracle.mamba_pool_oracle import MambaPoolOracle  # checker and CPU baseline only

            n_layers = 2  # bounded sample
            ref = MambaPoolOracle(2 * batch, n_layers, [[(3, 8192)]] * n_layers, [(hv, d, d)] * n_layers)
            for t in ref.temporal:
                t[...] = 1.0
            t1 = time.perf_counter()
            ref.copy_batched(np.arange(1, batch + 1), np.arange(batch + 1, 2 * batch + 1))
            dt = time.perf_counter() - t1
            row["cpu_port_GBps"] = moved * n_layers / layers / dt / 1e9
            row["cpu_sample"] = f"{n_layers} of {layers} layers, numpy port, 1 core"
        log(f"[state pool] {name}: {row['us_mean']:.1f} us mean ({row['us_min']:.1f} min)  "
            f"{row['achieved_GBps']:.0f} GB/s ({row['hbm_frac']*100:.1f}% of hbm peak)  "
            f"cpu {row.get('cpu_port_GBps', float('nan')):.2f} GB/s  bit exact {exact}")
        rows_out.append(row)
        del pool
    return rows_out


def run_decode_step_graph(dev, steps: int, warmup: int):
    """One decode step of one layer at shape 1's sizes (metadata build -> fused norm + rope + store
    -> decode attention: launch-bound), issued eagerly from Python and replayed from a HIP graph
    captured once.  Both run the same kernels on the same buffers."""
    import torch

    from mini_sglang_amd_kernel import (build_attention_metadata, paged_decode_attention,
                                        qk_norm_rope_store)

    n_q, n_kv, d, max_seq, slots = 16, 8, 128, 2048, 16384
    lens = [37, 128, 500, 1023]
    b = len(lens)
    g = torch.Generator().manual_seed(0x5EED0400)
    bf = lambda *s: torch.randn(s, generator=g).to(dev, torch.bfloat16)
    kc, vc, q, k, v = bf(slots, n_kv, d), bf(slots, n_kv, d), bf(b, n_q, d), bf(b, n_kv, d), bf(b, n_kv, d)
    qw, kw = torch.ones(d, dtype=torch.bfloat16, device=dev), torch.ones(d, dtype=torch.bfloat16, device=dev)
    table = torch.randperm(slots, generator=g)[:b * max_seq].to(torch.int32).view(b, max_seq).to(dev)
    rows = torch.arange(b, dtype=torch.int32, device=dev)
    start = torch.tensor(lens, dtype=torch.int32, device=dev)
    kv_lens = start.clone()
    out = torch.zeros(b, n_q, d, dtype=torch.bfloat16, device=dev)

    def step():
        meta = build_attention_metadata(table, rows, kv_lens, total_kv=b * max_seq)
        out_loc = table[rows.long(), (kv_lens - 1).long()]
        q_rot = qk_norm_rope_store(q, k, v, qw, kw, meta["positions"], out_loc, kc, vc, eps=1e-6,
                                   rope_base=1e6)
        out.copy_(paged_decode_attention(q_rot, kc, vc, meta["kv_indptr"], meta["kv_indices"],
                                         meta["num_kv_splits"], d ** -0.5, 32))

    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream(dev).wait_stream(side)
    torch.cuda.synchronize()
    eager_ms, _, eager_wall = time_steps(step, steps, warmup)
    want = out.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    out.zero_()
    graph_ms, _, graph_wall = time_steps(graph.replay, steps, warmup)
    torch.cuda.synchronize()
    row = {"sizes": "shape1_decode_step_one_layer", "batch": b, "eager_us": eager_ms * 1e3,
           "eager_wall_us": eager_wall / steps * 1e3, "graph_replay_us": graph_ms * 1e3,
           "graph_replay_wall_us": graph_wall / steps * 1e3, "same_bits": bool(torch.equal(out, want))}
    log(f"[decode step] eager {row['eager_us']:.1f} us on the device ({row['eager_wall_us']:.1f} wall), "
        f"graph replay {row['graph_replay_us']:.1f} us ({row['graph_replay_wall_us']:.1f} wall), "
        f"same bits {row['same_bits']}")
    return row


def run_radix_cache(cpu_baseline: bool):
    """Host-side prefix cache: 2048 finished requests (one of 8 shared 1024-token system prompts
    plus a 512-token body of their own) are inserted, then every request comes back with 64 new
    tokens and is matched.  Timed with the host clock; no GPU work.  The same trace through the
    pure-Python oracle (a quarter of it) is the CPU baseline."""
    import torch

    from mini_sglang_amd.kvcache import RadixCacheManager

    g = torch.Generator().manual_seed(0x5EED0200)
    prompts = torch.randint(0, 150000, (8, 1024), generator=g, dtype=torch.int32)
    bodies = torch.randint(0, 150000, (2048, 512 + 64), generator=g, dtype=torch.int32)
    which = torch.randint(0, 8, (2048,), generator=g)
    seqs = [torch.cat([prompts[int(which[i])], bodies[i]]) for i in range(2048)]
    pages = torch.arange(1536, dtype=torch.int32)

    def trace(insert, match, n):
        t0 = time.perf_counter()
        for i in range(n):
            insert(seqs[i][:1536], pages)
        t1 = time.perf_counter()
        hit = 0
        for i in range(n):
            hit += match(seqs[i])
        t2 = time.perf_counter()
        return (t1 - t0) / n, (t2 - t1) / n, hit / n

    mgr = RadixCacheManager()
    ins_s, match_s, hit = trace(mgr.insert_prefix, lambda s: mgr.match_prefix(s)[0].cached_len, 2048)
    row = {"requests": 2048, "tokens_per_request": 1536, "insert_us": ins_s * 1e6,
           "match_us": match_s * 1e6, "mean_cached_len": hit,
           "match_tokens_per_s": 1600 / match_s}
    if cpu_baseline:
        from oracle.radix_oracle import RadixOracle  # checker and CPU baseline only

        ora = RadixOracle(time.monotonic_ns)
        lists = [s.tolist() for s in seqs[:512]]
        page_list = pages.tolist()
        t0 = time.perf_counter()
        for ids in lists:
            ora.insert_prefix(ids[:1536], page_list)
        t1 = time.perf_counter()
        hit_o = sum(ora.match_prefix(ids)[0] for ids in lists)
        t2 = time.perf_counter()
        row["cpu_port_insert_us"] = (t1 - t0) / 512 * 1e6
        row["cpu_port_match_us"] = (t2 - t1) / 512 * 1e6
        row["cpu_port_sample"] = "first 512 requests, pure-Python oracle on lists, 1 core"
        row["agrees_with_oracle"] = bool(
            hit_o == sum(RadixCacheManager.match_prefix(mgr, s)[0].cached_len for s in seqs[:512]))
    log(f"[radix cache] insert {row['insert_us']:.1f} us  match {row['match_us']:.1f} us per request "
        f"(cached {hit:.0f} of 1600 tokens)  cpu port insert "
        f"{row.get('cpu_port_insert_us', float('nan')):.0f} us match "
        f"{row.get('cpu_port_match_us', float('nan')):.0f} us")
    return row


def run_small_launch_extends(dev, steps: int, warmup: int):
    """Extends too small to fill the chip (one long request, a short chunk): the tile kernels with
    their keys in one pass (knob 1) against the library's own choice of key splits.  Not one of the
    benchmark shapes; shows what the split buys and that both give the same result."""
    import torch

    from mini_sglang_amd.workloads import build_workload
    from mini_sglang_amd_kernel import _lib, paged_prefill_attention

    rows = []
    for name, prefix, extend, n_q, n_kv, d in (
            ("one_request_128k_context_1024_extend", 130048, 1024, 16, 4, 128),
            ("one_request_128k_context_1024_extend_head_dim_256", 130048, 1024, 16, 4, 256),
            ("one_request_32k_context_512_extend", 32768, 512, 32, 8, 128),
            ("one_request_8k_context_64_extend", 8192, 64, 32, 8, 128)):
        wl = build_workload(name, "prefill", seed=7, n_q=n_q, n_kv=n_kv, head_dim=d,
                            kv_lens=[prefix + extend], extend_lens=[extend], pool_factor=1.0,
                            pool_device=dev)
        g = wl.to(dev)

        def step():
            return paged_prefill_attention(g.q, g.k_cache, g.v_cache, g.qo_indptr, g.kv_indptr,
                                           g.kv_indices, g.prefix_lens, g.sm_scale, extend)
        row = {"sizes": name, "n_q": n_q, "n_kv": n_kv, "head_dim": d,
               "algorithmic_flops": wl.attention_flops()}
        outs = {}
        for label, knob in (("one_pass", 1), ("key_split", 0)):
            _lib.set_tuning(_lib.TUNE_PREFILL_KEY_SPLITS, knob)
            try:  # whatever happens, the later legs run with the library's own choice
                ms, _, _ = time_steps(step, max(3, steps // 5), max(1, warmup // 5))
                outs[label] = step().float()
                torch.cuda.synchronize()
            finally:
                _lib.set_tuning(_lib.TUNE_PREFILL_KEY_SPLITS, 0)
            row[label + "_us"] = ms * 1e3
            row[label + "_TFLOPs"] = row["algorithmic_flops"] / (ms * 1e-3) / 1e12
        row["max_abs_diff"] = float((outs["one_pass"] - outs["key_split"]).abs().max())
        log(f"[small launch] {name}: one pass {row['one_pass_us']:.0f} us, key split "
            f"{row['key_split_us']:.0f} us ({row['key_split_TFLOPs']:.0f} TFLOP/s), "
            f"max diff {row['max_abs_diff']:.1e}")
        rows.append(row)
        del g, wl
    return rows


def run_few_long_requests_decode(dev, steps: int, warmup: int):
    """Decode with one long request alone on the chip, or beside short ones: every workgroup's
    partial belongs to the same request, so the merge sees up to a hundred items per row.  Not
    one of the benchmark shapes; time per step and the rate over the K/V bytes of the step."""
    from mini_sglang_amd.workloads import build_workload

    rows = []
    for name, lens in (("one_request_8k", [8192]), ("one_request_32k", [32768]),
                       ("one_request_128k", [131072]),
                       ("one_request_100k_beside_31_of_1k", [100000] + [1024] * 31)):
        wl = build_workload(name, "decode", seed=7, n_q=32, n_kv=8, kv_lens=lens, pool_device=dev)
        g = wl.to(dev)
        ms, _, _ = time_steps(make_step(g), steps, warmup)
        row = {"sizes": name, "n_q": 32, "n_kv": 8, "head_dim": 128, "us": ms * 1e3,
               "algorithmic_bytes": wl.attention_bytes(),
               "achieved_TBps": wl.attention_bytes() / (ms * 1e-3) / 1e12}
        log(f"[few long requests] {name}: {row['us']:.1f} us, {row['achieved_TBps']:.2f} TB/s")
        rows.append(row)
        del g, wl
    return rows


def run_reference_microbench_shapes(dev, steps: int, warmup: int):
    """The shapes of the reference's own micro-benchmarks (one sequence, head_dim 256, its four
    head configurations, nine lengths: `test_and_bench/paged_prefill_attention.py:18-25, 267` with
    prefix 0, `paged_decode_attention.py:17-24, 288`), in microseconds per call.  The reference
    prints these beside MLX's dense SDPA and ships no recorded output, so there is no ratio to
    quote: the numbers are here for whoever runs the reference's scripts on their own machine."""
    from mini_sglang_amd.workloads import build_workload

    lens = (1, 237, 512, 809, 1024, 2048, 3333, 4096, 8192)
    rows = []
    for kind in ("prefill", "decode"):
        for n_kv, n_q in ((2, 16), (4, 16), (4, 24), (2, 32)):
            us = []
            for length in lens:
                wl = build_workload("m", kind, seed=7, n_q=n_q, n_kv=n_kv, head_dim=256,
                                    kv_lens=[length],
                                    extend_lens=[length] if kind == "prefill" else None,
                                    pool_device=dev)
                g = wl.to(dev)
                ms, _, _ = time_steps(make_step(g), max(3, steps // 2), max(1, warmup // 2),
                                      spinup_ms=10.0)
                us.append(round(ms * 1e3, 1))
                del g, wl
            rows.append({"kind": kind, "head_dim": 256, "n_kv": n_kv, "n_q": n_q,
                         "lengths": list(lens), "us": us})
            log(f"[reference shapes] {kind} kv {n_kv} q {n_q}: " +
                "  ".join(f"{n}:{u}" for n, u in zip(lens, us)))
    return rows


PROBE_SRC = os.path.join(ROOT, "bench_probes.hip")
PROBE_LIB = os.path.join(ROOT, "bench_probes.so")


def build_probes(force: bool = False) -> str:
    """Compile bench_probes.hip (the measurement aids below) into bench_probes.so beside this
    file.  hipcc cross-compiles for gfx950, so this also runs where there is no GPU."""
    import subprocess

    if force or not os.path.exists(PROBE_LIB) or os.path.getmtime(PROBE_SRC) > os.path.getmtime(PROBE_LIB):
        cmd = [os.environ.get("HIPCC", "/opt/rocm/bin/hipcc"), "--offload-arch=gfx950", "-O3",
               "-std=c++17", "-fPIC", "-fvisibility=hidden", "-Xclang", "-target-feature", "-Xclang",
               "-packed-fp32-ops", "-shared", PROBE_SRC, "-o", PROBE_LIB]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed for bench_probes.hip:\n{proc.stderr}")
    return PROBE_LIB


def _probe_lib():
    import ctypes

    return ctypes.CDLL(build_probes())


def hbm_read_probe(gib: int = 4, reps: int = 5):
    """A plain streaming read of `gib` GiB (16 bytes per lane and load, consecutive lanes on
    consecutive addresses, far beyond the 256 MB Infinity Cache): the rate the memory system
    gives a kernel that does nothing but read, beside the datasheet's 8 TB/s."""
    import ctypes

    lib = _probe_lib()
    lib.msgl_probe_hbm_read.restype = ctypes.c_int
    lib.msgl_probe_hbm_read.argtypes = [ctypes.c_size_t, ctypes.c_int, ctypes.POINTER(ctypes.c_double),
                                        ctypes.POINTER(ctypes.c_double)]
    best, mean = ctypes.c_double(0), ctypes.c_double(0)
    rc = lib.msgl_probe_hbm_read(gib << 30, reps, ctypes.byref(best), ctypes.byref(mean))
    if rc != 0:
        return None
    log(f"[hbm read probe] {gib} GiB x {reps}: best {best.value:.3f} TB/s, mean {mean.value:.3f} TB/s")
    return {"unit": "TB/s", "bytes": gib << 30, "reps": reps, "best": best.value, "mean": mean.value,
            "frac_of_datasheet_peak": mean.value * 1e12 / HBM_PEAK,
            "kernel": "grid-stride read, 16 B per lane and load, 8 loads in flight per lane"}


def mfma_rate_probe():
    """Sustained v_mfma_f32_32x32x16_bf16 rate of the whole chip on register-resident operands,
    nothing else running: all-zero operands and N(0,1) operands that change every instruction;
    then the random stream with the A operand of every instruction read from LDS (1 KB per MFMA,
    the way the attention kernels receive K and V).  The board lowers its shader clock to hold
    its power limit and MFMA power grows with the number of toggling operand bits, so the
    second and third figures are context for the prefill number; `roofline.frac` stays the
    fraction of the datasheet peak."""
    import ctypes

    lib = _probe_lib()
    lib.msgl_probe_mfma_rate.restype = ctypes.c_int
    lib.msgl_probe_mfma_rate.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_double),
                                         ctypes.POINTER(ctypes.c_double)]
    out = {"unit": "TFLOP/s", "kernel": "back-to-back v_mfma_f32_32x32x16_bf16, 4 waves per CU"}
    for name, mode in (("zero_operands", 0), ("random_operands", 1), ("random_operands_a_from_lds", 2)):
        tf, ghz = ctypes.c_double(0), ctypes.c_double(0)
        rc = lib.msgl_probe_mfma_rate(mode, 40000, ctypes.byref(tf), ctypes.byref(ghz))
        if rc != 0:
            return None if mode < 2 else out
        out[name] = tf.value
        out[name + "_shader_ghz"] = ghz.value
        log(f"[mfma probe] {name}: {tf.value:.0f} TFLOP/s at {ghz.value:.2f} GHz")
    return out


def issue_rate_probes():
    """LDS read rates and the issue rates of MFMA and VALU work on one and two waves per SIMD
    (bench_probes.hip): the machine figures that the extend kernels' schedules are read against."""
    import ctypes

    lib = _probe_lib()
    lib.msgl_probe_issue_rates.restype = ctypes.c_int
    lib.msgl_probe_issue_rates.argtypes = [ctypes.POINTER(ctypes.c_double), ctypes.c_int]
    out = (ctypes.c_double * 10)()
    if lib.msgl_probe_issue_rates(out, 10) != 0:
        return None
    res = {
        "lds_bytes_per_clk_per_cu": {"ds_read_b128": out[0], "ds_read_b64_tr_b16": out[1]},
        "simd_cycles_per_mfma_one_wave_per_simd": {"valu_0": out[2], "valu_4": out[3], "valu_8": out[4], "valu_16": out[5]},
        "simd_cycles_per_mfma_two_waves_per_simd": {"valu_0": out[6], "valu_8": out[7], "valu_16": out[8],
                                                    "valu_4_exp_1": out[9]},
    }
    log(f"[issue probe] LDS per CU and clock: ds_read_b128 {out[0]:.0f} B, ds_read_b64_tr_b16 {out[1]:.0f} B")
    log("[issue probe] SIMD cycles per v_mfma_f32_32x32x16_bf16 with K v_fma_f32 behind each, one wave per "
        f"SIMD: K=0 {out[2]:.1f}  K=4 {out[3]:.1f}  K=8 {out[4]:.1f}  K=16 {out[5]:.1f}; two waves per SIMD "
        f"(first start to last end): K=0 {out[6]:.1f}  K=8 {out[7]:.1f}  K=16 {out[8]:.1f}  "
        f"K=4 and one v_exp_f32 {out[9]:.1f}")
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-extra-shapes", action="store_true",
                    help="skip the legs on shapes outside the benchmark set (small launches, few long "
                         "requests, the reference's micro-benchmark shapes)")
    ap.add_argument("--configs", default="2,3,1,5,5w,4,3h")
    ap.add_argument("--no-check", action="store_true", help="skip the oracle comparison")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--tune", action="append", default=[], metavar="KNOB=VALUE",
                    help="set a msgl_set_tuning knob (benchmarking only), e.g. 0=512")
    ap.add_argument("--copy-probe-mib", type=int, default=0,
                    help="also run one device-to-device copy of this many MiB (a kernel of "
                         "known traffic that calibrates rocprofv3 FETCH_SIZE / WRITE_SIZE)")
    ap.add_argument("--no-metadata", action="store_true",
                    help="skip the figures of the kernels either side of the path: on-device metadata "
                         "build (slot table -> CSR arrays) and fused q/k norm + rope + KV-store")
    ap.add_argument("--no-mfma-probe", action="store_true",
                    help="skip the measurement aids: the matrix pipe's sustained rate on zero "
                         "and on random operands, and the rate of a plain streaming read of 4 GiB")
    ap.add_argument("--issue-probes", action="store_true",
                    help="also measure LDS read rates and MFMA / VALU issue rates (a second of GPU time)")
    ap.add_argument("--cpu-flops", type=float, default=3e11,
                    help="flop budget of the CPU baseline sample per shape")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs the hot path on ONE GPU; --gpus N with N > 1 is "
                 "not supported (no collective or sharding code is part of it)")

    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py: no ROCm GPU visible")
    from mini_sglang_amd_kernel import _lib

    _lib.load()  # fail loudly if the HIP library was not built
    for kv in args.tune:
        knob, value = kv.split("=")
        _lib.set_tuning(int(knob), int(value))
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    traffic = load_traffic()
    if args.copy_probe_mib > 0:
        n = args.copy_probe_mib << 20
        src = torch.empty(n, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)  # reads n bytes, writes n bytes
        torch.cuda.synchronize()
        log(f"[copy probe] {args.copy_probe_mib} MiB device copy done")
        del src, dst

    rows = []
    for tok in [t.strip() for t in args.configs.split(",") if t.strip()]:
        # "5w": shape 5 with the sliding window; "3h": shape 3 at head_dim 256
        suffix = {"w": "window", "h": "head_dim_256"}.get(tok[-1], "")
        cfg, variant = (int(tok[:-1]), suffix) if suffix else (int(tok), "")
        steps = args.steps if cfg != 4 else max(5, args.steps // 5)
        budget = 0.0 if args.no_cpu_baseline else args.cpu_flops
        row = run_config(cfg, variant, steps, args.warmup if cfg != 4 else max(2, args.warmup // 3),
                         not args.no_check, budget, dev)
        rows.append(row)
        perf = (f"{row['achieved_TBps']:.3f} TB/s" if row["bound"] == "hbm"
                else f"{row['achieved_TFLOPs']:.1f} TFLOP/s")
        clock = f"  shader clock {row['shader_ghz']:.2f} GHz" if row.get("shader_ghz") else ""
        log(f"[cfg {tok}] {row['workload']}: {row['ms_mean']*1e3:.1f} us mean "
            f"({row['ms_min']*1e3:.1f} min)  {perf}  {row['roofline_frac']*100:.1f}% of "
            f"{row['bound']} peak{clock}  err max {row.get('max_abs_err', float('nan')):.2e} "
            f"mean {row.get('mean_abs_err', float('nan')):.2e}  cpu "
            f"{row.get('cpu_baseline', {}).get('value', float('nan')):.4f} "
            f"{row.get('cpu_baseline', {}).get('unit', '')}")

    def find(cfg, variant_window=False):
        for r in rows:
            if (r["config"] == cfg and (r["sliding_window"] > 0) == variant_window
                    and r["head_dim"] == 128):
                return r
        return None

    head = find(2) or next((r for r in rows if r["bound"] == "hbm"), rows[0])
    pre = find(3)

    def roofline_obj(r):
        if r["bound"] == "hbm":
            return {"bound": "hbm", "achieved": r["achieved_TBps"] * 1e3, "peak": HBM_PEAK / 1e9,
                    "unit": "GB/s", "frac": r["roofline_frac"],
                    "traffic": traffic.get(r["workload"])}
        return {"bound": "mfma", "achieved": r["achieved_TFLOPs"], "peak": MFMA_PEAK / 1e12,
                "unit": "TFLOP/s", "frac": r["roofline_frac"], "traffic": traffic.get(r["workload"])}

    def cpu_obj(r):
        c = r.get("cpu_baseline")
        if not c:
            return None
        return {"value": c["value"], "unit": c["unit"], "cores": c["cores"], "kind": c["kind"],
                "sample": c["sample"]}

    result = {
        "metric": METRIC,
        "value": head.get("achieved_TBps", head.get("achieved_TFLOPs")),
        "unit": "TB/s" if head["bound"] == "hbm" else "TFLOP/s",
        "n_gpus": 1, "steps": head["steps"], "warmup": head["warmup"],
        "ms_per_step": head["ms_mean"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{head['workload']}: paged GQA decode, batch {head['batch']}, "
                               f"{head['n_q']} q / {head['n_kv']} kv heads, head_dim "
                               f"{head['head_dim']}, page size {head['page_size']}, "
                               f"{head['total_kv_tokens']} kv tokens, bf16 pool",
                   "parallelism": "1 GPU"},
        "roofline": roofline_obj(head),
        "cpu_baseline": cpu_obj(head),
    }
    if pre is not None:
        result["prefill"] = {
            "workload": f"{pre['workload']}: 8 requests x 512-token causal extend on cached "
                        f"prefixes, {pre['n_q']} q / {pre['n_kv']} kv heads, KV-store included",
            "value": pre["achieved_TFLOPs"], "unit": "TFLOP/s", "ms_per_step": pre["ms_mean"],
            "roofline": roofline_obj(pre), "cpu_baseline": cpu_obj(pre),
            "parity_ok": pre.get("parity_ok"), "kv_pool_bit_exact": pre.get("kv_pool_bit_exact"),
        }
        if not args.no_mfma_probe:
            probe = mfma_rate_probe()
            result["prefill"]["mfma_rate_probe"] = probe
            if probe and probe.get("random_operands"):
                # the same MFMA instruction issued back to back on random operands, on this box,
                # now: what the board sustains under its power limit
                result["prefill"]["frac_of_measured_mfma_rate"] = pre["achieved_TFLOPs"] / probe["random_operands"]
            if probe and probe.get("random_operands_a_from_lds"):
                result["prefill"]["frac_of_measured_lds_fed_mfma_rate"] = (
                    pre["achieved_TFLOPs"] / probe["random_operands_a_from_lds"])
    if not args.no_mfma_probe:
        result["hbm_read_probe"] = hbm_read_probe()
    if args.issue_probes:
        result["issue_probes"] = issue_rate_probes()
    if not args.no_metadata:
        result["qk_norm_rope_store"] = run_norm_rope_store(dev, args.steps, args.warmup,
                                                           not args.no_cpu_baseline)
        result["gdn_state_inplace"] = run_gdn_state(dev, args.steps, args.warmup,
                                                    not args.no_cpu_baseline)
        result["metadata_build"] = run_metadata_build(dev, args.steps, args.warmup,
                                                      not args.no_cpu_baseline)
        result["radix_prefix_cache"] = run_radix_cache(not args.no_cpu_baseline)
        result["decode_step_graph"] = run_decode_step_graph(dev, args.steps, args.warmup)
        result["state_pool_copy"] = run_state_pool(dev, args.steps, args.warmup, not args.no_cpu_baseline)
        if not args.no_extra_shapes:
            result["small_launch_extends"] = run_small_launch_extends(dev, args.steps, args.warmup)
            result["few_long_requests_decode"] = run_few_long_requests_decode(dev, args.steps, args.warmup)
            result["reference_microbench_shapes"] = run_reference_microbench_shapes(dev, args.steps, args.warmup)
    result["all_configs"] = rows
    print(json.dumps(result))


if __name__ == "__main__":
    main()

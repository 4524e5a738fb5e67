#!/usr/bin/env python3
"""Headline benchmark: DeepSeek-V3-shape absorbed-MLA paged decode, bf16, one MI355X.

A step = one layer's decode attention for the whole batch: the latent-KV cache write of the new
tokens, the split-KV decode kernel and the split reduction, inputs resident in HBM.  Prints ONE JSON
line with the metric (us/layer, lower is better), the roofline of the dominant kernel (the split-KV
decode kernel, timed on its own with HIP events on the launch stream) and a CPU baseline (the oracle
on a bounded sample of the same workload, on the host cores of this box).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0           # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0  # dense bf16


def host_cpu():
    """Model name and logical CPU count of the host, and the thread count the oracle runs with (the GPU box gives one GPU's
    job 16 CPUs whatever the host has)."""
    model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    logical = os.cpu_count() or 1
    return model, logical, min(logical, 16)


def cpu_fields():
    model, logical, threads = host_cpu()
    torch.set_num_threads(threads)
    return {"cores": threads, "host_logical_cpus": logical, "cpu_model": model}


# the acceptance bars of attention outputs against the fp32 oracle: (max-abs, mean-rel = sum|err| / sum|ref|)
PARITY_BARS = {"bf16": (2e-2, 2e-3), "fp8": (6e-2, 6e-3)}


def parity_fields(err: torch.Tensor, ref: torch.Tensor, kind: str, **extra) -> dict:
    """max-abs and mean-relative error of an attention output next to the bar of its cache type, and whether it is met."""
    max_abs, mean_rel = err.max().item(), (err.sum() / ref.abs().sum().clamp_min(1e-30)).item()
    bar = PARITY_BARS[kind]
    return {"max_abs": round(max_abs, 5), "mean_rel": round(mean_rel, 6), "bar": {"max_abs": bar[0], "mean_rel": bar[1]},
            "parity_ok": bool(max_abs <= bar[0] and mean_rel <= bar[1]), **extra}


def gemm_probe(dev) -> dict:
    """torch.matmul of square bf16 matrices, 50 queued calls between one pair of events, after a ramp of the clock."""
    out = {}
    for n in (4096, 8192):
        for name, make in (("normal", lambda: torch.randn(n, n, device=dev).bfloat16()), ("zeros", lambda: torch.zeros(n, n, device=dev, dtype=torch.bfloat16))):
            a, b_ = make(), make()
            f = lambda: torch.matmul(a, b_)
            clock_ramp(f, 0.2, 5)
            s_, e_ = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            s_.record()
            for _ in range(50):
                f()
            e_.record()
            torch.cuda.synchronize()
            out[f"{n}^3 {name}"] = round(2 * n ** 3 * 50 / (s_.elapsed_time(e_) * 1e-3) / 1e12, 1)
            del a, b_
    return out


def median3(fn):
    ts, res = [], None
    for _ in range(3):
        t0 = time.perf_counter()
        res = fn()
        ts.append(time.perf_counter() - t0)
    return sorted(ts)[1], res


def clock_ramp(fn, seconds=0.3, batch=20):
    """Keep the GPU busy with `fn`, untimed, before a measurement.  The part leaves its low-power state over tens of
    milliseconds of work: the decode step measures 183 us right after seconds of host-side set-up and 145 a moment later."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(batch):
            fn()
        torch.cuda.synchronize()


def _hwmon(name):
    import glob
    hits = sorted(glob.glob(f"/sys/class/drm/card*/device/hwmon/hwmon*/{name}"))
    return hits[0] if hits else None


def _read_watts(path):
    try:
        with open(path) as f:
            return int(f.read()) / 1e6
    except (OSError, ValueError):
        return None


def socket_power(fn, seconds=2.0, batch=20):
    """Socket power (hwmon power1_input, sampled every 50 ms by a host thread) while `fn` is queued back to back for
    `seconds`, the first half second left out; None where the driver exposes no such file.  Says whether the timed kernel
    runs at the part's power cap, where fewer cycles buy a lower clock instead of less time."""
    import threading
    src, cap = _hwmon("power1_input"), _hwmon("power1_cap")
    if src is None or _read_watts(src) is None:
        return None
    samples, stop = [], threading.Event()
    t0 = time.perf_counter()

    def sampler():
        while not stop.is_set():
            w = _read_watts(src)
            if w is not None and time.perf_counter() - t0 > 0.5:
                samples.append(w)
            time.sleep(0.05)
    th = threading.Thread(target=sampler)
    th.start()
    calls = 0
    a, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    while time.perf_counter() - t0 < seconds:
        for _ in range(batch):
            fn()
        torch.cuda.synchronize()
        calls += batch
    e.record()
    torch.cuda.synchronize()
    stop.set()
    th.join()
    if not samples:
        return None
    us = a.elapsed_time(e) * 1e3 / calls
    watts = sum(samples) / len(samples)
    return {"socket_w_avg": round(watts, 1), "socket_w_max": round(max(samples), 1),
            "cap_w": _read_watts(cap) if cap else None, "seconds": seconds, "us_per_launch": round(us, 2),
            "mj_per_launch": round(watts * us * 1e-3, 1), "source": "hwmon power1_input, 50 ms samples"}


def profile_traffic(fname, applies=True):
    """HBM bytes per launch of the roofline kernel as the committed counter summary states them (a line
    `traffic_bytes_per_launch = N` in profiles/<fname>); None when the summary is absent or the run is not the workload it
    was taken on.  A counter run cannot be made from inside this script."""
    if not applies:
        return None, None
    import re
    try:
        with open(os.path.join(ROOT, "profiles", fname)) as f:
            m = re.search(r"^traffic_bytes_per_launch\s*=\s*([0-9_]+)", f.read(), re.M)
    except OSError:
        return None, None
    return (int(m.group(1).replace("_", "")), "profiles/" + fname) if m else (None, None)


def build_workload(seed: int, batch: int, heads: int, lo: int, hi: int, q_len: int):
    from oracle import mla_oracle as O       # input generator only (bits identical for oracle and GPU)
    return O.make_decode_case(batch, heads, lo, hi, seed=seed, q_len=q_len)


def algorithmic_bytes(case, heads):
    lens = case["seq_lens"].long()
    b = lens.numel()
    t = b * case["q_len"]
    kv = int(lens.sum()) * 576 * 2
    q = t * heads * 576 * 2
    o = t * heads * 512 * 2
    wr = t * 576 * 2
    tables = 4 * (int(((lens + 127) // 128).sum()) + 2 * b)
    return dict(kv=kv, q=q, out=o, cache_write=wr, tables=tables, total=kv + q + o + wr + tables)


def bench_dsa(K, dev, args):
    """configs[3]: lightning indexer (64 fp8 heads x 128) over contexts uniform[32768, 65536], batch 32, top-2048,
    sparse absorbed MLA over the selected rows.  Index keys and queries are N(0,1) values put through the per-token e4m3
    quantiser (the keys by the product's quantising cache write, a sequence at a time).  Per-stage device times (HIP events
    on the launch stream); a sample of sequences is recomputed by the oracle, timed, and compared."""
    from oracle import mla_oracle as O
    g = torch.Generator().manual_seed(args.seed)
    B, H, N, k = 32, 64, 128, 2048
    lens = torch.randint(32768, 65537, (B,), generator=g).to(torch.int32)
    nblk_seq = (lens + 127) // 128
    nblk = int(nblk_seq.sum())
    perm = torch.randperm(nblk, generator=g)
    bt = torch.zeros(B, int(nblk_seq.max()), dtype=torch.int32)
    o = 0
    for b in range(B):
        n = int(nblk_seq[b])
        bt[b, :n] = perm[o:o + n].to(torch.int32)
        o += n
    btd, lensd = bt.to(dev), lens.to(dev)
    sample = (0, B - 1)
    k8 = torch.zeros(nblk, 128, 128, dtype=torch.uint8, device=dev)
    ks = torch.zeros(nblk, 128, dtype=torch.float32, device=dev)
    k_src = {}
    torch.manual_seed(args.seed)
    for b in range(B):
        L = int(lens[b])
        x = torch.randn(L, 128, device=dev).bfloat16()
        pos = torch.arange(L, device=dev)
        K.quant_rows_fp8(x, k8, ks, slot_mapping=btd[b, pos // 128].long() * 128 + pos % 128)
        if b in sample:
            k_src[b] = x.cpu()
    q8c, qsc = O.fp8_quant_token(torch.randn(B, H, 128, generator=g))
    wc = torch.randn(B, H, generator=g)
    q8, w = q8c.to(dev), (wc * qsc).to(dev)            # the caller folds the query scale into the head weights
    nope = torch.randn(nblk, 128, 512, device=dev).bfloat16()
    rope = torch.randn(nblk, 128, 64, device=dev).bfloat16()
    qnc, qrc = torch.randn(B, N, 512, generator=g).bfloat16(), torch.randn(B, N, 64, generator=g).bfloat16()
    qn, qr = qnc.to(dev), qrc.to(dev)
    max_len = int(lens.max())
    logits = torch.empty(B, K.indexer_logits_stride(max_len), device=dev)
    idx = torch.empty(B, k, dtype=torch.int32, device=dev)
    rows = torch.empty(B, k, dtype=torch.int32, device=dev)
    counts = torch.empty(B, dtype=torch.int32, device=dev)
    out = torch.empty(B, N, 512, dtype=torch.bfloat16, device=dev)
    splits = args.splits or K.default_num_splits(B, 1, N, k)
    scale = 192 ** -0.5
    stages = [
        ("indexer", lambda: K.indexer_scores(q8, w, k8, ks, btd, lensd, logits, max_seq_len=max_len)),
        ("topk_with_rows", lambda: K.topk(logits, lensd, k, idx, block_table=btd, page_size=128, num_pages=nblk, rows=rows,
                                          counts=counts)),
        # counts come from K.topk on this row list, so they cannot exceed its width: no clamp launch, as in the backend
        ("sparse_decode", lambda: K.sparse_decode(qn, qr, nope, rope, rows, counts, scale, out, num_splits=splits,
                                                  counts_bounded=True)),
    ]

    def whole():
        for _, f in stages:
            f()

    def ev_time(fn, n):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        a, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(n):
            fn()
        e.record()
        torch.cuda.synchronize()
        return a.elapsed_time(e) * 1e3 / n

    clock_ramp(whole)
    total = ev_time(whole, args.steps)
    # the chain again as one captured HIP graph
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        whole()
        with torch.cuda.graph(graph, stream=side):
            whole()
    torch.cuda.synchronize()
    clock_ramp(graph.replay)                                  # (the capture left the queue idle)
    total_graph = ev_time(graph.replay, args.steps)
    # a stage timed alone in a launch loop is bounded below by the host's launch rate (about 10 us a call): the small
    # stages read high here, the per-kernel durations of a rocprofv3 kernel trace are the better figure for them
    per_stage = {name: round(ev_time(f, args.steps), 2) for name, f in stages}
    sum_l = int(lens.sum())
    idx_bytes = sum_l * (128 + 4) + B * H * (128 + 4) + sum_l * 4          # fp8 keys + scales, queries + weights, logits out
    sparse_bytes = B * k * 576 * 2 + B * N * (576 + 512) * 2
    ideal_us = (idx_bytes + sum_l * 4 + sparse_bytes) / (HBM_PEAK_GBS * 1e9) * 1e6
    best = total_graph                                        # the serving path replays whole steps from graphs
    traffic, traffic_src = profile_traffic("dsa_chain_b32_ctx32k_64k.md", args.seed == 0)
    res = {
        "metric": "DSA decode us/layer (B=32, ctx 32k-64k, indexer 64 fp8 heads + top-2048 + sparse MLA 128 heads)",
        "value": round(best, 2), "unit": "us/layer", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "higher_is_better": False, "dtype": "fp8 (indexer) / bf16 (attention)",
        "data": "synthetic: N(0,1) index keys / queries quantised per token to e4m3, N(0,1) bf16 latent cache",
        "config": {"workload": "configs[3]: DSA sparse decode path", "batch": B, "index_heads": H, "heads": N, "topk": k,
                   "seq_lens": "uniform[32768,65536]", "sum_seq_len": sum_l, "kv_splits": splits, "seed": args.seed},
        "chain_us": {"eager_launches": round(total, 2), "hip_graph_replay": round(total_graph, 2)},
        "stage_us_launch_loop": per_stage,
        "roofline": {"kernel": "dsa_indexer_fp8_kernel", "bound": "hbm",
                     "achieved": round(idx_bytes / (per_stage["indexer"] * 1e-6) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(idx_bytes / (per_stage["indexer"] * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
                     "traffic": traffic, "traffic_source": traffic_src, "algorithmic_bytes": idx_bytes},
        "chain_roofline": {"hbm_bytes": idx_bytes + sum_l * 4 + sparse_bytes, "ideal_us_at_8TBs": round(ideal_us, 2),
                           "frac": round(ideal_us / best, 4)},
    }
    if args.no_cpu_baseline:
        return res
    # oracle chain of the sampled sequences on the host: logits of every visible key, stable top-k, attention over the picks
    cpu = cpu_fields()
    whole()
    torch.cuda.synchronize()
    lg, idx_c = logits.cpu(), idx.cpu()
    worst_logit, sets_equal, t_cpu = 0.0, True, 0.0
    att_err, att_ref = [], []
    for b in sample:
        L = int(lens[b])
        ref8, ref_s = O.fp8_quant_token(k_src[b])
        r = rows[b].long()
        small_n = nope.view(-1, 512)[r].cpu().view(k // 128, 128, 512)
        small_r = rope.view(-1, 64)[r].cpu().view(k // 128, 128, 64)

        def chain():
            sc = O.indexer_scores(q8c[b], qsc[b], ref8, ref_s, wc[b])
            picks = O.topk_stable(sc, k, L)
            att = O.sparse_decode(qnc[b:b + 1], qrc[b:b + 1], small_n, small_r, torch.arange(k // 128, dtype=torch.int32)[None],
                                  torch.tensor([k], dtype=torch.int32), torch.arange(k, dtype=torch.int32)[None], scale)
            return sc, picks, att
        t, (sc, picks, att) = median3(chain)
        t_cpu += t
        worst_logit = max(worst_logit, ((lg[b, :L] - sc).abs().max() / sc.abs().max()).item())
        sets_equal &= idx_c[b].tolist() == sorted(O.topk_stable(lg[b], k, L).tolist())
        att_err.append((out[b:b + 1].float().cpu() - att).abs())
        att_ref.append(att)
    sample_l = sum(int(lens[b]) for b in sample)
    res["cpu_baseline"] = {"value": round(t_cpu * sum_l / sample_l * 1e6, 1), "unit": "us/layer", **cpu, "kind": "port",
                           "sample": f"oracle chain (indexer logits, stable top-k, sparse attention; torch fp32) of sequences "
                                     f"{list(sample)} of {B} ({sample_l} of {sum_l} keys), median of 3 each, scaled by key count",
                           "sample_seconds": round(t_cpu, 3)}
    att = parity_fields(torch.cat(att_err), torch.cat(att_ref), "bf16")
    res["gpu_vs_oracle"] = {"logits_max_err_rel_to_row_max": worst_logit, "topk_sets_equal_stable_topk_of_gpu_logits": sets_equal,
                            "attention": att, "sequences": list(sample),
                            "parity_ok": bool(att["parity_ok"] and sets_equal and worst_logit <= 2e-3)}
    res["parity_ok"] = res["gpu_vs_oracle"]["parity_ok"]
    return res


def bench_prefill(K, dev, args):
    """configs[2]: non-absorbed chunked prefill, 4 sequences, a 2048-token query chunk each over 16384 cached tokens,
    128 heads (qk 128 + 64 rope, v 128).  Times the attention kernels (context part, then the causal suffix continuing
    from the context's result: no merge launch) and, beside them, the separate merge the reference's flow has, the latent
    gather and the torch GEMM that up-projects the latent to K/V."""
    g = torch.Generator().manual_seed(args.seed)
    B, N, Q, C = 4, 128, 2048, 16384
    scale = 192 ** -0.5
    bf = lambda *shape: torch.randn(*shape, generator=g).bfloat16().to(dev)
    qn, qp = bf(B * Q, N, 128), bf(B * Q, N, 64)
    # suffix (the chunk's own keys) and context (the cached prefix), already up-projected
    ks_n, ks_p, vs = bf(B * Q, N, 128), bf(B * Q, 64), bf(B * Q, N, 128)
    kc_n = torch.randn(B * C, N, 128, device=dev).bfloat16()
    kc_p = torch.randn(B * C, 64, device=dev).bfloat16()
    vc = torch.randn(B * C, N, 128, device=dev).bfloat16()
    cu_q = torch.arange(0, (B + 1) * Q, Q, dtype=torch.int32, device=dev)
    cu_c = torch.arange(0, (B + 1) * C, C, dtype=torch.int32, device=dev)
    o_s = torch.empty(B * Q, N, 128, dtype=torch.float32, device=dev)      # partials that the merge reads stay fp32
    o_c = torch.empty_like(o_s)
    o = torch.empty(B * Q, N, 128, dtype=torch.bfloat16, device=dev)
    o_m = torch.empty_like(o)
    l_s = torch.empty(B * Q, N, dtype=torch.float32, device=dev)
    l_c = torch.empty_like(l_s)
    # latent cache of the prefix for the gather + up-projection leg
    pages = B * C // 128
    nope = torch.randn(pages, 128, 512, device=dev).bfloat16()
    rope = torch.randn(pages, 128, 64, device=dev).bfloat16()
    bt = torch.randperm(pages, generator=g).to(torch.int32).view(B, C // 128).to(dev)
    gathered = torch.empty(B * C, 576, dtype=torch.bfloat16, device=dev)
    w_up = (torch.randn(512, N * 256, generator=g) * 0.02).bfloat16().to(dev)

    # `value` is timed on bf16 keys and values, as the configuration states them.  Beside it: the same numbers handed over as
    # fp16 (every bf16 draw is an fp16 number), which is what the backend does when the model's up-projection is a plain
    # weight - it makes keys and values with an fp16 GEMM, and the kernel then converts no value tile.
    h = lambda x: x.to(torch.float16)
    kc_n16, kc_p16, vc16, ks_n16, ks_p16, vs16 = h(kc_n), h(kc_p), h(vc), h(ks_n), h(ks_p), h(vs)
    stages = [
        ("context_attention", lambda: K.prefill_varlen(qn, qp, kc_n, kc_p, vc, cu_q, cu_c, Q, scale, False, o_c, l_c)),
        ("suffix_attention", lambda: K.prefill_varlen(qn, qp, ks_n, ks_p, vs, cu_q, cu_q, Q, scale, True, o, prev_out=o_c,
                                                      prev_lse=l_c)),
        ("suffix_attention_alone", lambda: K.prefill_varlen(qn, qp, ks_n, ks_p, vs, cu_q, cu_q, Q, scale, True, o_s, l_s)),
        ("context_attention_fp16_kv", lambda: K.prefill_varlen(qn, qp, kc_n16, kc_p16, vc16, cu_q, cu_c, Q, scale, False, o_c, l_c)),
        ("suffix_attention_fp16_kv", lambda: K.prefill_varlen(qn, qp, ks_n16, ks_p16, vs16, cu_q, cu_q, Q, scale, True, o_m,
                                                              prev_out=o_c, prev_lse=l_c)),
        ("merge_as_a_launch_of_its_own", lambda: K.merge_states(o_c, l_c, o_s, l_s, o_m)),
        ("gather_latent", lambda: K.gather_paged(nope, rope, gathered, bt, cu_c, B)),
        ("kv_up_proj_torch_gemm", lambda: torch.matmul(gathered[:, :512], w_up)),
        ("kv_up_proj_torch_gemm_fp16", lambda: torch.matmul(h(gathered[:, :512]), h(w_up))),
    ]

    def ev_time(fn, n):
        for _ in range(2):
            fn()
        torch.cuda.synchronize()
        a, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(n):
            fn()
        e.record()
        torch.cuda.synchronize()
        return a.elapsed_time(e) * 1e3 / n

    n = max(3, min(args.steps, 10))
    per = {name: round(ev_time(f, n), 1) for name, f in stages}
    fl_c = B * N * Q * C * 2 * (192 + 128)
    fl_s = B * N * Q * (Q + 1) // 2 * 2 * (192 + 128)
    attn_us = per["context_attention"] + per["suffix_attention"]
    traffic, traffic_src = profile_traffic("mla_prefill_varlen_4x2048_over_16k.md", args.seed == 0)
    extra = {}
    if not args.no_cpu_baseline:
        # one (sequence, head) pair recomputed by the oracle as a single causal attention over prefix + chunk keys
        from oracle import mla_oracle as O
        cpu = cpu_fields()
        sb, sh = 1, 5
        c = lambda x: x.float().cpu().bfloat16()
        kq = slice(sb * Q, (sb + 1) * Q)
        kc = slice(sb * C, (sb + 1) * C)
        k_n = torch.cat([c(kc_n[kc, sh:sh + 1]), c(ks_n[kq, sh:sh + 1])])
        k_p = torch.cat([c(kc_p[kc]), c(ks_p[kq])])
        v_a = torch.cat([c(vc[kc, sh:sh + 1]), c(vs[kq, sh:sh + 1])])
        q_n, q_p = c(qn[kq, sh:sh + 1]), c(qp[kq, sh:sh + 1])
        t_cpu, (ref, _) = median3(lambda: O.attention_varlen(q_n, q_p, k_n, k_p, v_a, [0, Q], [0, C + Q], scale, True))
        err = (o[kq, sh:sh + 1].float().cpu() - ref).abs()
        extra["cpu_baseline"] = {"value": round(t_cpu * B * N * 1e6, 1), "unit": "us/layer", **cpu, "kind": "port",
                                 "sample": f"oracle attention_varlen (torch fp32) of 1 of {B * N} (sequence, head) pairs: {Q} "
                                           f"query rows over {C + Q} keys, median of 3, scaled by pair count",
                                 "sample_seconds": round(t_cpu, 3)}
        extra["gpu_vs_oracle"] = parity_fields(err, ref, "bf16", pair=[sb, sh])
        extra["parity_ok"] = extra["gpu_vs_oracle"]["parity_ok"]
    return {
        **extra,
        "metric": "MLA chunked prefill us/layer (4 x 2048-token chunk over 16384 cached tokens, 128 heads, bf16, attention kernels)",
        "value": round(attn_us, 1), "unit": "us/layer", "n_gpus": 1, "steps": n, "warmup": 2, "higher_is_better": False,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "configs[2]: non-absorbed chunked prefill", "sequences": B, "chunk": Q, "prefix": C, "heads": N,
                   "seed": args.seed},
        "stage_us": per,
        "with_fp16_keys_values_us": round(per["context_attention_fp16_kv"] + per["suffix_attention_fp16_kv"], 1),
        "roofline": {"kernel": "mla_prefill_varlen_kernel", "bound": "mfma",
                     "achieved": round((fl_c + fl_s) / ((per["context_attention"] + per["suffix_attention"]) * 1e-6) / 1e12, 1),
                     "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round((fl_c + fl_s) / ((per["context_attention"] + per["suffix_attention"]) * 1e-6) / 1e12
                                   / MFMA_BF16_PEAK_TFLOPS, 4),
                     "traffic": traffic, "traffic_source": traffic_src, "algorithmic_flops": fl_c + fl_s,
                     "socket_power": None if args.no_power_probe else socket_power(stages[0][1], batch=4)},
    }


def bench_fp8(K, dev, args):
    """configs[4]: fp8-e4m3 block-scaled latent cache, batch 256, contexts uniform[16384, 32768], 128 heads, q_len 2
    (MTP pair), page 128; a step = fp8 cache write of the 512 new tokens + decode, replayed as a captured HIP graph."""
    g = torch.Generator().manual_seed(args.seed)
    B, N, QL = 256, 128, 2
    lens = torch.randint(16384, 32769, (B,), generator=g).to(torch.int32)
    nblk_seq = (lens + 127) // 128
    nblk = int(nblk_seq.sum())
    perm = torch.randperm(nblk, generator=g).to(torch.int32)
    bt = torch.zeros(B, int(nblk_seq.max()), dtype=torch.int32)
    o = 0
    for b in range(B):
        n = int(nblk_seq[b])
        bt[b, :n] = perm[o:o + n]
        o += n
    cache = torch.zeros(nblk, 128, K.FP8_ROW_BYTES, dtype=torch.uint8, device=dev)
    # fill the cache on the GPU through the product's own quantising write, a sequence at a time; sequence 0 keeps its
    # source rows for the oracle
    torch.manual_seed(args.seed)
    btd = bt.to(dev)
    for b in range(B):
        L = int(lens[b])
        c_b, r_b = torch.randn(L, 512, device=dev).bfloat16(), torch.randn(L, 64, device=dev).bfloat16()
        pos = torch.arange(L, device=dev)
        K.cache_write_fp8(c_b, r_b, btd[b, pos // 128].long() * 128 + pos % 128, cache)
        if b == 0:
            src0 = (c_b.cpu(), r_b.cpu())
    T = B * QL
    qn = torch.randn(T, N, 512, device=dev).bfloat16()
    qr = torch.randn(T, N, 64, device=dev).bfloat16()
    new_c = torch.randn(T, 512, device=dev).bfloat16()
    new_r = torch.randn(T, 64, device=dev).bfloat16()
    slots = torch.empty(T, dtype=torch.int64)
    for b in range(B):
        for j in range(QL):
            pos = int(lens[b]) - QL + j
            slots[b * QL + j] = int(bt[b, pos // 128]) * 128 + pos % 128
    slots, lensd = slots.to(dev), lens.to(dev)
    out = torch.empty(T, N, 512, dtype=torch.bfloat16, device=dev)
    splits = args.splits or K.default_num_splits(B, QL, N, int(lens.max()))

    def step():
        K.cache_write_fp8(new_c, new_r, slots, cache)
        K.decode_fp8(qn, qr, cache, btd, lensd, 192 ** -0.5, out, q_len=QL, num_splits=splits)

    for _ in range(2):
        step()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()

    def ev_time(fn, n):
        fn()
        torch.cuda.synchronize()
        a, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(n):
            fn()
        e.record()
        torch.cuda.synchronize()
        return a.elapsed_time(e) * 1e3 / n

    n = max(3, min(args.steps, 10))
    clock_ramp(graph.replay, batch=4)                         # (the capture left the queue idle)
    t_graph = ev_time(graph.replay, n)
    clock_ramp(step, batch=4)
    t_eager = ev_time(step, n)
    sum_l = int(lens.sum())
    flops = sum_l * N * QL * 2 * (576 + 512)
    bytes_ = sum_l * K.FP8_ROW_BYTES + T * N * (576 + 512) * 2
    best = t_graph                                            # configs[4] is quoted on the replayed graph
    traffic, traffic_src = profile_traffic("mla_decode_fp8_b256_ctx16k_32k.md", args.seed == 0)
    extra = {}
    if not args.no_cpu_baseline:
        # sequence 0 on the host: the oracle's block quantiser on the same source rows, then the oracle's decode
        from oracle import mla_oracle as O
        cpu = cpu_fields()
        L = int(lens[0])
        c0, r0 = src0[0].clone(), src0[1].clone()
        c0[L - QL:], r0[L - QL:] = new_c[:QL].cpu(), new_r[:QL].cpu()
        q8, sc = O.fp8_quant_block(c0.float())
        npg = (L + 127) // 128
        deq, rp = torch.zeros(npg * 128, 512), torch.zeros(npg * 128, 64, dtype=torch.bfloat16)
        deq[:L], rp[:L] = O.fp8_dequant_block(q8, sc), r0
        qn0, qr0 = qn[:QL].cpu(), qr[:QL].cpu()
        t_cpu, ref = median3(lambda: O.absorbed_decode(qn0, qr0, deq.view(npg, 128, 512), rp.view(npg, 128, 64),
                                                       torch.arange(npg, dtype=torch.int32)[None], lens[:1], 192 ** -0.5))
        err = (out[:QL].float().cpu() - ref).abs()
        extra["cpu_baseline"] = {"value": round(t_cpu * sum_l / L * 1e6, 1), "unit": "us/layer", **cpu, "kind": "port",
                                 "sample": f"oracle absorbed_decode (torch fp32, cache rows dequantised beforehand) of sequence 0 of "
                                           f"{B} ({L} of {sum_l} cached tokens), median of 3, scaled by token count",
                                 "sample_seconds": round(t_cpu, 3)}
        extra["gpu_vs_oracle"] = parity_fields(err, ref, "fp8", sequence=0)
        extra["parity_ok"] = extra["gpu_vs_oracle"]["parity_ok"]
    return {
        **extra,
        "metric": "MLA decode us/layer, fp8-e4m3 block-scaled cache (B=256, ctx 16k-32k, 128 heads, q_len 2)",
        "value": round(best, 1), "unit": "us/layer", "n_gpus": 1, "steps": n, "warmup": 3, "higher_is_better": False,
        "dtype": "bf16 MFMA over fp8 storage (dequantised on chip)", "data": "synthetic",
        "config": {"workload": "configs[4]: fp8 cache, high-batch MTP decode", "batch": B, "heads": N, "q_len": QL,
                   "seq_lens": "uniform[16384,32768]", "sum_seq_len": sum_l, "kv_splits": splits, "seed": args.seed},
        "step_us": {"hip_graph_replay": round(t_graph, 1), "eager_launches": round(t_eager, 1)},
        "roofline": {"kernel": "mla_decode_v3_fp8_kernel<false, 4>", "bound": "mfma", "achieved": round(flops / (best * 1e-6) / 1e12, 1),
                     "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(flops / (best * 1e-6) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
                     "traffic": traffic, "traffic_source": traffic_src,
                     "algorithmic_flops": flops, "algorithmic_bytes": bytes_,
                     "hbm_gbs": round(bytes_ / (best * 1e-6) / 1e9, 1),
                     "socket_power": None if args.no_power_probe else socket_power(step, batch=4)},
    }


def bench_prologue(K, dev, args):
    """The step in front of the path: fused RMSNorm + rotary embedding + cache write of T new tokens and the rotary embedding
    of their 128 query heads, at decode size (T = 64: latency) and at prefill-chunk size (T = 8192: bandwidth)."""
    import time
    from oracle import mla_oracle as O
    g = torch.Generator().manual_seed(args.seed)
    N = 128
    out = {}
    cpu = None
    for T in (64, 8192):
        kv = torch.randn(T, 576, generator=g).bfloat16()
        gamma = (1 + 0.1 * torch.randn(512, generator=g)).bfloat16()
        pos = torch.randint(0, 32768, (T,), generator=g)
        cos, sin = O.rope_tables(pos)
        nblk = T // 128 + 64
        slots = torch.randperm(nblk * 128, generator=g)[:T]
        q = torch.randn(T, N, 192, generator=g).bfloat16()
        d = [x.to(dev) for x in (kv, gamma, cos, sin, slots, q)]
        nope = torch.zeros(nblk, 128, 512, dtype=torch.bfloat16, device=dev)
        rope = torch.zeros(nblk, 128, 64, dtype=torch.bfloat16, device=dev)
        q_out = torch.empty(T, N, 64, dtype=torch.bfloat16, device=dev)

        def fused():
            K.kv_rmsnorm_rope_cache(d[0], d[1], d[2], d[3], d[4], nope, rope, eps=1e-6)

        def qrope():
            K.interleave_rope(d[5][..., 128:], d[2], d[3], out=q_out)

        def ev_time(fn, n, reps=10):
            # `reps` launches per replay of a captured graph: a launch loop from Python would measure the host (tens of
            # microseconds a call), not these kernels
            fn()
            torch.cuda.synchronize()
            side = torch.cuda.Stream()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.stream(side):
                fn()
                with torch.cuda.graph(graph, stream=side):
                    for _ in range(reps):
                        fn()
            torch.cuda.synchronize()
            for _ in range(2):
                graph.replay()
            torch.cuda.synchronize()
            a, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(n):
                graph.replay()
            e.record()
            torch.cuda.synchronize()
            return a.elapsed_time(e) * 1e3 / (n * reps)

        t_f, t_q = ev_time(fused, args.steps), ev_time(qrope, args.steps)
        kv_bytes = T * (1152 + 2 * 128 + 8 + 1152) + 1024           # kv in, cos + sin rows, slot, cache rows out, gamma
        q_bytes = T * N * 128 * 2 + T * 2 * 128
        out[T] = {"fused_kv_us": round(t_f, 2), "q_rope_us": round(t_q, 2), "fused_kv_gbs": round(kv_bytes / t_f / 1e3, 1),
                  "q_rope_gbs": round(q_bytes / t_q / 1e3, 1), "kv_bytes": kv_bytes, "q_bytes": q_bytes}
        if T == 8192:
            nope_c, rope_c = torch.zeros(nblk, 128, 512).bfloat16(), torch.zeros(nblk, 128, 64).bfloat16()
            ts = []
            for _ in range(3):
                t0 = time.perf_counter()
                O.kv_rmsnorm_rope_cache(kv, gamma, cos, sin, slots, nope_c, rope_c, 1e-6)
                O.interleave_rope(q[..., 128:], cos, sin)
                ts.append(time.perf_counter() - t0)
            cpu = sorted(ts)[1]
            got = nope.cpu().view(-1, 512)[slots]
            bits = (got.view(torch.int16).int() - nope_c.view(-1, 512)[slots].view(torch.int16).int()).abs().max().item()
    big = out[8192]
    step_us = big["fused_kv_us"] + big["q_rope_us"]
    tot_bytes = big["kv_bytes"] + big["q_bytes"]
    return {
        "metric": "fused RMSNorm + rotary embedding + cache write, plus query rotary embedding, us (T = 8192 tokens, 128 heads)",
        "value": round(step_us, 2), "unit": "us", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "higher_is_better": False, "dtype": "bf16 (fp32 arithmetic)", "data": "synthetic",
        "config": {"workload": "step before the attention path: fused norm + rotary + cache write", "tokens": [64, 8192], "heads": N, "seed": args.seed},
        "sizes": {str(k): v for k, v in out.items()},
        "roofline": {"kernel": "kv_rmsnorm_rope_cache_kernel<false> + interleave_rope_kernel", "bound": "hbm",
                     "achieved": round(tot_bytes / step_us / 1e3, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(tot_bytes / step_us / 1e3 / HBM_PEAK_GBS, 4), "traffic": None,
                     "algorithmic_bytes": tot_bytes},
        "cpu_baseline": {"value": round(cpu * 1e6, 1), "unit": "us", **cpu_fields(),
                         "kind": "port", "sample": "oracle (torch float64) on the same 8192 tokens, median of 3",
                         "gpu_vs_oracle_max_ulp": int(bits)},
        "parity_ok": bool(bits <= 1),                         # at most one bf16 ulp from the float64 oracle
    }


def bench_epilogue(K, dev, args):
    """The step behind the split kernel: merge of the split-KV partials + value up-projection into the layer's [T, N*128]
    output, on the headline shape (B=64, 128 heads, contexts 4k-8k, 4 chunks per sequence).  Fused (one launch) beside the
    reference's sequence (merge, batched GEMM, transpose, copy), each timed as HIP-graph replays of the part after the
    split kernel (the split kernel runs once, outside the timed region: its partials stay in the workspace)."""
    import time
    from oracle import mla_oracle as O
    B, N = 64, 128
    case = build_workload(args.seed, B, N, 4096, 8192, 1)
    g = {k: (v.to(dev) if torch.is_tensor(v) else v) for k, v in case.items()}
    gen = torch.Generator().manual_seed(args.seed + 1)
    w_cpu = (torch.randn(N, 512, 128, generator=gen) * 0.02).bfloat16()
    w = w_cpu.to(dev)
    splits = args.splits or K.default_num_splits(B, 1, N, int(case["seq_lens"].max()))
    ws = torch.zeros(K._lib.load().mla_decode_workspace_bytes(B, 1, N, splits), dtype=torch.uint8, device=dev)
    o = torch.empty(N, B, 512, dtype=torch.bfloat16, device=dev)
    out_f = torch.empty(B, N * 128, dtype=torch.bfloat16, device=dev)
    out_u = torch.empty_like(out_f)
    dargs = (g["q_nope"], g["q_rope"], g["nope"], g["rope"], g["block_table"], g["seq_lens"], case["scale"])
    K.decode(*dargs, o.transpose(0, 1), num_splits=splits, workspace=ws, phase="split")
    torch.cuda.synchronize()

    def fused():
        K.decode(*dargs, out_f, num_splits=splits, workspace=ws, phase="reduce", w_uv=w)

    def unfused():
        K.decode(*dargs, o.transpose(0, 1), num_splits=splits, workspace=ws, phase="reduce")
        out_u.copy_(torch.bmm(o, w).transpose(0, 1).contiguous().view(-1, N * 128))

    def ev_time(fn, n, reps=10):
        fn()
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            fn()
            with torch.cuda.graph(graph, stream=side):
                for _ in range(reps):
                    fn()
        torch.cuda.synchronize()
        for _ in range(2):
            graph.replay()
        torch.cuda.synchronize()
        a, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(n):
            graph.replay()
        e.record()
        torch.cuda.synchronize()
        return a.elapsed_time(e) * 1e3 / (n * reps)

    t_f, t_u = ev_time(fused, args.steps), ev_time(unfused, args.steps)
    segments = B * (splits + 1)                               # upper bound of the partials the merge reads
    alg_bytes = segments * N * 1040 + N * 512 * 128 * 2 + B * N * 128 * 2
    # oracle chain on the host: attention of a sample of sequences, then the up-projection of all
    sample = 8
    cpu_info = cpu_fields()
    t0 = time.perf_counter()
    ref_o = O.absorbed_decode(case["q_nope"][:sample], case["q_rope"][:sample], case["nope"], case["rope"],
                              case["block_table"][:sample], case["seq_lens"][:sample], case["scale"])
    ref = torch.bmm(ref_o.transpose(0, 1), w_cpu.float()).transpose(0, 1).reshape(sample, N * 128)
    cpu_s = time.perf_counter() - t0
    err = (out_f[:sample].float().cpu() - ref).abs().max().item()
    same = (out_f.float() - out_u.float()).abs().max().item()
    traffic, traffic_src = profile_traffic("mla_reduce_vup_b64_128heads.md", args.seed == 0 and not args.splits)
    return {
        "metric": "merge of the split-KV partials + value up-projection, us/layer (B=64, 128 heads, 4 chunks per sequence)",
        "value": round(t_f, 2), "unit": "us/layer", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "higher_is_better": False, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "step behind the split kernel: merge + W_UV up-projection into [T, N*128]", "batch": B, "heads": N,
                   "kv_splits": splits, "seed": args.seed},
        "unfused_us": round(t_u, 2), "fused_vs_unfused_max_abs": same,
        "roofline": {"kernel": "mla_reduce_vup_kernel", "bound": "hbm", "achieved": round(alg_bytes / t_f / 1e3, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(alg_bytes / t_f / 1e3 / HBM_PEAK_GBS, 4),
                     "traffic": traffic, "traffic_source": traffic_src, "algorithmic_bytes": alg_bytes},
        "cpu_baseline": {"value": round(cpu_s * B / sample * 1e6, 1), "unit": "us/layer", **cpu_info,
                         "kind": "port", "sample": f"oracle attention (torch fp32) of {sample} of {B} sequences + up-projection, scaled by sequence count",
                         "gpu_vs_oracle_max_abs": err},
        "parity_ok": bool(err <= 2e-2),                       # max-abs bar of a bf16 attention output
    }


def bench_layer(K, dev, args):
    """The attention part of one decode layer the way the backend runs it (the classes a vLLM worker would call, on the
    headline shape): fused RMSNorm + rotary embedding + cache write of the new tokens, rotary embedding of the query,
    then ``NPUMLAImpl.forward`` = absorption GEMM, split-KV kernel, merge fused with the value up-projection into the
    layer's [T, N*128] output.  Timed as queued eager launches and as HIP-graph replays."""
    import time
    from types import SimpleNamespace
    from oracle import mla_oracle as O
    from omni_npu_amd import _vllm_compat as V
    from omni_npu_amd.attention.backends import mla
    B, N, EPS = args.batch, args.heads, 1e-6
    case = build_workload(args.seed, B, N, args.len_lo, args.len_hi, 1)
    lens = case["seq_lens"]
    gen = torch.Generator().manual_seed(args.seed + 7)
    w_kv_b = (torch.randn(512, N * 256, generator=gen) * 0.05).bfloat16()
    q = torch.randn(B, N, 192, generator=gen).bfloat16()
    kv = torch.randn(B, 576, generator=gen).bfloat16()
    gamma = (1 + 0.1 * torch.randn(512, generator=gen)).bfloat16()
    cos, sin = O.rope_tables(lens.long() - 1)
    impl = mla.NPUMLAImpl(num_heads=N, head_size=576, scale=192 ** -0.5, num_kv_heads=1, alibi_slopes=None,
                          sliding_window=None, kv_cache_dtype="auto", logits_soft_cap=None,
                          attn_type=V.AttentionType.DECODER, kv_sharing_target_layer_name=None, q_lora_rank=None,
                          kv_lora_rank=512, qk_nope_head_dim=128, qk_rope_head_dim=64, qk_head_dim=192, v_head_dim=128,
                          kv_b_proj=lambda x: (x @ w_kv_b.to(x.device),))
    kvw = w_kv_b.view(512, N, 256)
    impl.W_UK_T = kvw[..., :128].permute(1, 2, 0).contiguous().to(dev)
    impl.W_UV = kvw[..., 128:].transpose(0, 1).contiguous().to(dev)
    qsl = torch.arange(B + 1, dtype=torch.int32)
    common = V.CommonAttentionMetadata(
        query_start_loc=qsl.to(dev), query_start_loc_cpu=qsl.clone(), seq_lens=lens.to(dev), seq_lens_cpu=lens.clone(),
        num_computed_tokens_cpu=lens - 1, num_reqs=B, num_actual_tokens=B, max_query_len=1, max_seq_len=int(lens.max()),
        block_table_tensor=case["block_table"].to(dev), slot_mapping=case["slot_mapping"].to(dev))
    cfg = SimpleNamespace(
        scheduler_config=SimpleNamespace(max_num_seqs=B), model_config=SimpleNamespace(max_model_len=16384, dtype=torch.bfloat16),
        cache_config=SimpleNamespace(block_size=128, cache_dtype="auto"),
        parallel_config=SimpleNamespace(cp_kv_cache_interleave_size=1, decode_context_parallel_size=1, worker_cls=None),
        compilation_config=SimpleNamespace(max_cudagraph_capture_size=B, pass_config=None), kv_transfer_config=None,
        speculative_config=None)
    builder = mla.NPUMLAMetadataBuilder(V.AttentionSpec(128, 1, 576, torch.bfloat16), ["layer"], cfg, dev)
    meta = builder.build(0, common)
    nope, rope = case["nope"].to(dev), case["rope"].to(dev)
    d_q, d_kv, d_gamma, d_cos, d_sin = (x.to(dev) for x in (q, kv, gamma, cos, sin))
    kvc = torch.empty(B, 512, dtype=torch.bfloat16, device=dev)
    kpe = torch.empty(B, 64, dtype=torch.bfloat16, device=dev)
    q_in = d_q.clone()
    out = torch.zeros(B, N * 128, dtype=torch.bfloat16, device=dev)

    def layer():
        K.kv_rmsnorm_rope_cache(d_kv, d_gamma, d_cos, d_sin, meta.slot_mapping, nope, rope, eps=EPS, kv_a_out=kvc, k_pe_out=kpe,
                                q_rope=d_q[..., 128:], q_out=q_in[..., 128:])
        impl.cache_written_for = (meta, B)
        impl.forward(None, q_in, kvc, kpe.unsqueeze(1), (nope, rope), meta, output=out)

    def timed(fn, n):
        a, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        a.record()
        for _ in range(n):
            fn()
        e.record()
        torch.cuda.synchronize()
        return a.elapsed_time(e) * 1e3 / n

    clock_ramp(layer)
    for _ in range(args.warmup):
        layer()
    t_eager = sorted(timed(layer, args.steps) for _ in range(3))[1]
    reps = 10
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        layer()
        with torch.cuda.graph(graph, stream=side):
            for _ in range(reps):
                layer()
    torch.cuda.synchronize()
    clock_ramp(graph.replay, batch=2)                         # (the capture left the queue idle)
    t_graph = sorted(timed(graph.replay, max(1, args.steps // reps)) for _ in range(3))[1] / reps

    # oracle chain on the host for a sample of sequences
    sample = min(8, B)
    cpu_info = cpu_fields()
    t0 = time.perf_counter()
    kv_a = O.rms_norm(kv[:, :512], gamma, EPS)
    k_pe = O.interleave_rope(kv[:, 512:], cos, sin)
    c_nope, c_rope = case["nope"].clone(), case["rope"].clone()
    O.cache_write(c_nope, case["slot_mapping"], kv_a)
    O.cache_write(c_rope, case["slot_mapping"], k_pe)
    q_pe = O.interleave_rope(q[:sample, :, 128:], cos[:sample], sin[:sample])
    ql = O.q_absorb(q[:sample, :, :128], impl.W_UK_T.cpu()).bfloat16()
    ref_o = O.absorbed_decode(ql, q_pe, c_nope, c_rope, case["block_table"][:sample], lens[:sample], impl.scale)
    ref = O.v_up_proj(ref_o.transpose(0, 1).contiguous().bfloat16(), impl.W_UV.cpu()).view(sample, -1)
    cpu_s = time.perf_counter() - t0
    err = (out[:sample].float().cpu() - ref.float()).abs().max().item()
    alg = algorithmic_bytes(case, N)
    alg_bytes = alg["kv"] + alg["cache_write"] + alg["tables"] + B * N * (192 + 128) * 2 + 2 * N * 128 * 512 * 2
    return {
        "metric": f"MLA decode attention of one layer through the backend classes, us/layer (B={B}, ctx {args.len_lo // 1024}k-{args.len_hi // 1024}k, {N} heads)",
        # (the serving path runs the layer from a captured graph: that figure is the value, the eager queue beside it)
        "value": round(t_graph, 2), "unit": "us/layer", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "higher_is_better": False, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "configs[1] through NPUMLAMetadataBuilder + NPUMLAImpl.forward: norm + rope + cache write, "
                               "query rope, absorption GEMM, split-KV decode, merge + W_UV", "batch": B, "heads": N,
                   "sum_seq_len": int(lens.sum()), "seed": args.seed},
        "layer_us": {"eager_launches_queued": round(t_eager, 2), "hip_graph_replay": round(t_graph, 2)},
        "roofline": {"kernel": "whole layer", "bound": "hbm", "achieved": round(alg_bytes / t_graph / 1e3, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(alg_bytes / t_graph / 1e3 / HBM_PEAK_GBS, 4),
                     "traffic": None, "algorithmic_bytes": alg_bytes},
        "cpu_baseline": {"value": round(cpu_s * B / sample * 1e6, 1), "unit": "us/layer", **cpu_info, "kind": "port",
                         "sample": f"oracle chain (torch fp32) of {sample} of {B} sequences, scaled by sequence count",
                         "gpu_vs_oracle_max_abs": err},
        "parity_ok": bool(err <= 2e-2),                       # max-abs bar of a bf16 attention output
    }


def bench_dsa_layer(K, dev, args):
    """The attention part of one DSA decode layer through the backend classes, on the configs[3] shape (B = 32, contexts
    uniform[32768, 65536], 64 fp8 index heads, top-2048, 128 heads): fused RMSNorm + rotary embedding + cache write + query
    rope, ``LightningIndexer`` (quantise q and the new index keys, key-cache write, fp8 scores, top-k with cache rows),
    ``NPUDSAImpl.forward`` (absorption GEMM, sparse split-KV kernel, merge fused with the value up-projection)."""
    import time
    from types import SimpleNamespace
    from oracle import mla_oracle as O
    from omni_npu_amd import _vllm_compat as V
    from omni_npu_amd.attention.backends import dsa
    B, H, N, k, EPS = 32, 64, 128, 2048, 1e-6
    g = torch.Generator().manual_seed(args.seed)
    lens = torch.randint(32768, 65537, (B,), generator=g).to(torch.int32)
    nblk_seq = (lens + 127) // 128
    nblk = int(nblk_seq.sum())
    perm = torch.randperm(nblk, generator=g)
    bt = torch.zeros(B, int(nblk_seq.max()), dtype=torch.int32)
    o = 0
    for b in range(B):
        n = int(nblk_seq[b])
        bt[b, :n] = perm[o:o + n].to(torch.int32)
        o += n
    btd = bt.to(dev)
    raw = torch.zeros(nblk * 128 * 704, dtype=torch.bfloat16, device=dev).view(torch.uint8)
    kv_cache = dsa.NPUDSABackend.reshape_kv_cache(raw, nblk, 128, 1, 704, dtype=torch.bfloat16)
    torch.manual_seed(args.seed)
    step_blk = 2048
    for b0 in range(0, nblk, step_blk):
        b1 = min(nblk, b0 + step_blk)
        kv_cache[0][b0:b1].copy_(torch.randn(b1 - b0, 128, 1, 512, device=dev))
        kv_cache[1][b0:b1].copy_(torch.randn(b1 - b0, 128, 1, 64, device=dev))
    k8v, ksv = dsa.indexer_cache_views(kv_cache[2])
    for b in range(B):
        L = int(lens[b])
        pos = torch.arange(L, device=dev)
        K.quant_rows_fp8(torch.randn(L, 128, device=dev).bfloat16(), k8v, ksv,
                         slot_mapping=btd[b, pos // 128].long() * 128 + pos % 128)
    slots = torch.stack([bt[b, (int(lens[b]) - 1) // 128].long() * 128 + (int(lens[b]) - 1) % 128 for b in range(B)])
    w_kv_b = (torch.randn(512, N * 256, generator=g) * 0.05).bfloat16()
    q = torch.randn(B, N, 192, generator=g).bfloat16()
    kv = torch.randn(B, 576, generator=g).bfloat16()
    gamma = (1 + 0.1 * torch.randn(512, generator=g)).bfloat16()
    iq, ik = torch.randn(B, H, 128, generator=g).bfloat16(), torch.randn(B, 128, generator=g).bfloat16()
    iw = torch.randn(B, H, generator=g)
    cos, sin = O.rope_tables(lens.long() - 1)
    cfg = SimpleNamespace(
        scheduler_config=SimpleNamespace(max_num_seqs=B), model_config=SimpleNamespace(max_model_len=65536, dtype=torch.bfloat16),
        cache_config=SimpleNamespace(block_size=128, cache_dtype="auto"),
        parallel_config=SimpleNamespace(cp_kv_cache_interleave_size=1, decode_context_parallel_size=1, worker_cls=None),
        compilation_config=SimpleNamespace(max_cudagraph_capture_size=B, pass_config=None), kv_transfer_config=None,
        speculative_config=None)
    impl = dsa.NPUDSAImpl(num_heads=N, head_size=576, scale=192 ** -0.5, num_kv_heads=1, alibi_slopes=None,
                          sliding_window=None, kv_cache_dtype="auto", logits_soft_cap=None,
                          attn_type=V.AttentionType.DECODER, kv_sharing_target_layer_name=None, q_lora_rank=None,
                          kv_lora_rank=512, qk_nope_head_dim=128, qk_rope_head_dim=64, qk_head_dim=192, v_head_dim=128,
                          kv_b_proj=lambda x: (x @ w_kv_b.to(x.device),))
    kvw = w_kv_b.view(512, N, 256)
    impl.W_UK_T = kvw[..., :128].permute(1, 2, 0).contiguous().to(dev)
    impl.W_UV = kvw[..., 128:].transpose(0, 1).contiguous().to(dev)
    indexer = dsa.LightningIndexer(k, H, 128, max_tokens=B, device=dev)
    impl.indexer = indexer
    qsl = torch.arange(B + 1, dtype=torch.int32)
    common = V.CommonAttentionMetadata(
        query_start_loc=qsl.to(dev), query_start_loc_cpu=qsl.clone(), seq_lens=lens.to(dev), seq_lens_cpu=lens.clone(),
        num_computed_tokens_cpu=lens - 1, num_reqs=B, num_actual_tokens=B, max_query_len=1, max_seq_len=int(lens.max()),
        block_table_tensor=btd, slot_mapping=slots.to(dev))
    builder = dsa.NPUDSAMetadataBuilder(V.AttentionSpec(128, 1, 704, torch.bfloat16), ["layer"], cfg, dev)
    meta = builder.build(0, common)
    d_q, d_kv, d_gamma, d_cos, d_sin, d_iq, d_ik, d_iw = (x.to(dev) for x in (q, kv, gamma, cos, sin, iq, ik, iw))
    kvc = torch.empty(B, 512, dtype=torch.bfloat16, device=dev)
    kpe = torch.empty(B, 64, dtype=torch.bfloat16, device=dev)
    q_in = d_q.clone()
    out = torch.zeros(B, N * 128, dtype=torch.bfloat16, device=dev)

    def layer():
        K.kv_rmsnorm_rope_cache(d_kv, d_gamma, d_cos, d_sin, meta.slot_mapping, kv_cache[0], kv_cache[1], eps=EPS, kv_a_out=kvc,
                                k_pe_out=kpe, q_rope=d_q[..., 128:], q_out=q_in[..., 128:])
        indexer(d_iq, d_ik, d_iw, kv_cache, meta)
        impl.cache_written_for = (meta, B)
        impl.forward(None, q_in, kvc, kpe.unsqueeze(1), kv_cache, meta, output=out)

    def timed(fn, n):
        a, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        a.record()
        for _ in range(n):
            fn()
        e.record()
        torch.cuda.synchronize()
        return a.elapsed_time(e) * 1e3 / n

    clock_ramp(layer)
    for _ in range(args.warmup):
        layer()
    t_eager = sorted(timed(layer, args.steps) for _ in range(3))[1]
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        layer()
        with torch.cuda.graph(graph, stream=side):
            layer()
    torch.cuda.synchronize()
    clock_ramp(graph.replay)                                  # (the capture left the queue idle)
    t_graph = sorted(timed(graph.replay, args.steps) for _ in range(3))[1]

    # oracle: sparse attention over the positions the GPU picked, on the caches as the GPU left them, for two sequences
    cpu_info = cpu_fields()
    sel = indexer.topk_indices_buffer[:B].cpu()
    checks, cpu_s = [], 0.0
    for b in (0, B - 1):
        L = int(lens[b])
        picks = sel[b][sel[b] >= 0]
        assert picks.numel() == min(k, L) and int(picks.max()) < L and picks.unique().numel() == picks.numel()
        pages = bt[b, :int(nblk_seq[b])].long()
        c_nope = kv_cache[0][pages.to(dev)].cpu().view(-1, 128, 512)
        c_rope = kv_cache[1][pages.to(dev)].cpu().view(-1, 128, 64)
        t0 = time.perf_counter()
        q_pe = O.interleave_rope(q[b:b + 1, :, 128:], cos[b:b + 1], sin[b:b + 1])
        ql = O.q_absorb(q[b:b + 1, :, :128], impl.W_UK_T.cpu()).bfloat16()
        local_bt = torch.arange(pages.numel(), dtype=torch.int32).view(1, -1)
        ref_o = O.sparse_decode(ql, q_pe, c_nope, c_rope, local_bt, [L], sel[b:b + 1], impl.scale)
        ref = O.v_up_proj(ref_o.transpose(0, 1).contiguous().bfloat16(), impl.W_UV.cpu()).view(-1)
        cpu_s += time.perf_counter() - t0
        checks.append((out[b].float().cpu() - ref.float()).abs().max().item())
    return {
        "metric": "DSA decode attention of one layer through the backend classes, us/layer (B=32, ctx 32k-64k, top-2048, 128 heads)",
        "value": round(t_graph, 2), "unit": "us/layer", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "higher_is_better": False, "dtype": "fp8 (indexer) / bf16 (attention)", "data": "synthetic",
        "config": {"workload": "configs[3] through NPUDSAMetadataBuilder + LightningIndexer + NPUDSAImpl.forward with the fused "
                               "prologue in front", "batch": B, "heads": N, "index_heads": H, "topk": k,
                   "sum_seq_len": int(lens.sum()), "seed": args.seed},
        "layer_us": {"eager_launches_queued": round(t_eager, 2), "hip_graph_replay": round(t_graph, 2)},
        "roofline": None,
        "cpu_baseline": {"value": round(cpu_s * B / 2 * 1e6, 1), "unit": "us/layer", **cpu_info, "kind": "port",
                         "sample": "oracle rope + absorption + sparse attention + up-projection (torch fp32) of 2 of 32 tokens on the "
                                   "GPU's picks, scaled by token count; the indexer is not in this sample",
                         "gpu_vs_oracle_max_abs": max(checks)},
        "parity_ok": bool(max(checks) <= 2e-2),
    }


def bench_window(K, dev, args):
    """Decode with static sink tokens and a sliding window (the reference's variant of attention/backends/mla.py:705-779):
    B=64, 128 heads, 4096-8192 keys behind a 128-key sink, window 4096.  One step = window plan + dense split kernel over
    the shortened sequences + merge, replayed as a HIP graph; the split kernel is also timed alone."""
    import time
    from oracle import mla_oracle as O
    B, N, sink, win = 64, 128, 128, 4096
    case = build_workload(args.seed, B, N, 4096, 8192, 1)
    nsb = sink // 128
    nblk = case["nope"].shape[0]
    gen = torch.Generator().manual_seed(args.seed + 2)
    sink_nope, sink_rope = torch.randn(nsb, 128, 512, generator=gen).bfloat16(), torch.randn(nsb, 128, 64, generator=gen).bfloat16()
    nope_c, rope_c = torch.cat([case["nope"], sink_nope]), torch.cat([case["rope"], sink_rope])
    bt_c = torch.cat([torch.arange(nblk, nblk + nsb, dtype=torch.int32).view(1, -1).expand(B, -1), case["block_table"]], 1).contiguous()
    nope, rope, bt, lens = nope_c.to(dev), rope_c.to(dev), bt_c.to(dev), case["seq_lens"].to(dev)
    qn, qr = case["q_nope"].to(dev), case["q_rope"].to(dev)
    out = torch.empty(B, N, 512, dtype=torch.bfloat16, device=dev)
    splits = args.splits or None

    def step():
        K.decode(qn, qr, nope, rope, bt, lens, case["scale"], out, num_splits=splits, sink_len=sink, window=win)

    for _ in range(max(args.warmup, 2)):
        step()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        step()
        with torch.cuda.graph(graph, stream=side):
            step()
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    ts = []
    for _ in range(args.steps):
        a, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        graph.replay()
        e.record()
        torch.cuda.synchronize()
        ts.append(a.elapsed_time(e) * 1e3)
    t_step = sum(ts) / len(ts)
    visible = int((torch.clamp(case["seq_lens"], max=win) + sink).sum())
    alg_bytes = visible * 1152 + B * N * 576 * 2 + B * N * 512 * 2
    sample = 4
    cpu_info = cpu_fields()
    t0 = time.perf_counter()
    ref = O.sink_decode(case["q_nope"][:sample], case["q_rope"][:sample], nope_c, rope_c, bt_c[:sample], case["seq_lens"][:sample],
                        sink, case["scale"], win)
    cpu_s = time.perf_counter() - t0
    err = (out[:sample].float().cpu() - ref).abs().max().item()
    traffic, traffic_src = profile_traffic("mla_decode_window_b64_sink128_w4096.md", args.seed == 0 and not args.splits)
    return {
        "metric": "MLA decode with static sink + sliding window, us/layer (B=64, ctx 4k-8k, sink 128, window 4096, 128 heads, bf16)",
        "value": round(t_step, 2), "unit": "us/layer", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "higher_is_better": False, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "static sink tokens + sliding window decode (plan + split + merge, graph replay)", "batch": B,
                   "heads": N, "sink_len": sink, "window": win, "visible_keys": visible, "seed": args.seed},
        "roofline": {"kernel": "mla_window_plan_kernel + mla_decode_v3_kernel<false, true, 4> + merge (whole step)", "bound": "hbm",
                     "achieved": round(alg_bytes / t_step / 1e3, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(alg_bytes / t_step / 1e3 / HBM_PEAK_GBS, 4),
                     "traffic": traffic, "traffic_source": traffic_src, "algorithmic_bytes": alg_bytes},
        "cpu_baseline": {"value": round(cpu_s * B / sample * 1e6, 1), "unit": "us/layer", **cpu_info,
                         "kind": "port", "sample": f"oracle sink_decode (torch fp32) of {sample} of {B} sequences, scaled by sequence count",
                         "gpu_vs_oracle_max_abs": err},
        "parity_ok": bool(err <= 2e-2),                       # max-abs bar of a bf16 attention output
    }


def finish(res: dict) -> None:
    """Prints the one JSON line and ends the process with status 1 when a comparison with the oracle missed its bar
    (``parity_ok`` false at the top level or in any secondary workload)."""
    print(json.dumps(res))
    sys.stdout.flush()
    bad = [name for name, r in [("", res)] + list(res.get("secondary", {}).items()) if r.get("parity_ok") is False]
    if bad:
        print(f"bench.py: parity bar missed ({', '.join(b or res.get('config', {}).get('workload', 'workload') for b in bad)})",
              file=sys.stderr)
        sys.exit(1)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--heads", type=int, default=128)
    ap.add_argument("--len-lo", type=int, default=4096)
    ap.add_argument("--len-hi", type=int, default=8192)
    ap.add_argument("--q-len", type=int, default=1)
    ap.add_argument("--splits", type=int, default=0, help="KV splits per sequence (0 = library default)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-power-probe", action="store_true",
                    help="decode, fp8 and prefill workloads: skip the two seconds of queued launches under the socket power reading")
    ap.add_argument("--graph", action="store_true",
                    help="decode workload: time the steps as replays of captured HIP graphs (--graph-layers steps per graph) "
                         "instead of eager launches; the default line carries the one-step-per-graph figure either way "
                         "(step_us.hip_graph_replay)")
    ap.add_argument("--graph-layers", type=int, default=10,
                    help="with --graph: steps captured into one HIP graph, as a model captures all its layers in one; the "
                         "largest divisor of --steps up to this number is used")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run a plain 512 MiB device copy three times: its known traffic calibrates the FETCH_SIZE / "
                         "WRITE_SIZE counters of a rocprofv3 --pmc run of this script")
    ap.add_argument("--workload", default="decode", choices=["decode", "dsa", "prefill", "fp8", "prologue", "epilogue", "window", "layer", "dsa-layer"],
                    help="decode = configs[1] (the headline metric); dsa = configs[3], per-stage times of the sparse path; prefill = configs[2], the chunked-prefill attention kernels; fp8 = configs[4], the quantised-cache decode; prologue = the fused norm + rotary + cache write in front of the path; epilogue = merge of the partials + value up-projection behind the split kernel; layer = the attention part of a decode layer through the backend classes (NPUMLAMetadataBuilder + NPUMLAImpl.forward with the fused steps around it); dsa-layer = the same for configs[3] (LightningIndexer + NPUDSAImpl.forward)")
    ap.add_argument("--l2-resident", action="store_true",
                    help="decode workload, a probe and not the workload: every block-table entry folded onto 8 pages, so the "
                         "cache rows come from L2 instead of HBM (same kernel, same instructions, same result check)")
    ap.add_argument("--gemm-probe", action="store_true",
                    help="decode workload: also time the vendor library's bf16 GEMM (torch.matmul, 4096^3 and 8192^3, N(0,1) and "
                         "all-zero operands) on this part: what its matrix pipes sustain under the same power cap")
    ap.add_argument("--cpu-seqs", type=int, default=64, help="sequences in the CPU-baseline sample")
    ap.add_argument("--no-secondary", action="store_true",
                    help="decode workload: leave out the short runs of configs[2], [3] and [4] that the default line carries "
                         "under \"secondary\" (they run after the headline measurement, outside its timed region)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (no sharding, no collectives); --gpus must be 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(2)

    from omni_npu_amd import kernels as K
    dev = torch.device("cuda:0")
    if args.copy_probe:
        src = torch.empty(512 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    others = {"dsa": bench_dsa, "prefill": bench_prefill, "fp8": bench_fp8, "prologue": bench_prologue,
              "epilogue": bench_epilogue, "window": bench_window, "layer": bench_layer, "dsa-layer": bench_dsa_layer}
    if args.workload in others:
        finish(others[args.workload](K, dev, args))
        return
    case = build_workload(args.seed, args.batch, args.heads, args.len_lo, args.len_hi, args.q_len)
    if args.l2_resident:
        case["block_table"] = case["block_table"] % 8        # (the oracle reads through the same table)
    heads, b, q_len = args.heads, args.batch, args.q_len
    t = b * q_len
    g = {k: (v.to(dev) if torch.is_tensor(v) else v) for k, v in case.items()}
    out = torch.empty(heads, t, 512, dtype=torch.bfloat16, device=dev)     # head-major, as the reference returns it
    out_v = out.transpose(0, 1)
    max_len = int(case["seq_lens"].max())
    splits = args.splits or K.default_num_splits(b, q_len, heads, max_len)
    ws = torch.empty(K._lib.load().mla_decode_workspace_bytes(b, q_len, heads, splits), dtype=torch.uint8, device=dev)

    def step():
        # cache write of the step's new tokens (inside the split kernel) + split-KV decode + merge: two launches
        K.decode(g["q_nope"], g["q_rope"], g["nope"], g["rope"], g["block_table"], g["seq_lens"], case["scale"], out_v,
                 q_len=q_len, num_splits=splits, workspace=ws, new_rows=(g["new_c"], g["new_r"], g["slot_mapping"]))

    eager_step = step
    # The timed region is args.steps steps, queued without a host wait in between, bracketed by synchronisations on the
    # host and by one pair of HIP events on the launch stream.  --graph replays them from captured HIP graphs (the
    # product's decode path can: compilation/acl_graph.py), `layers` steps per graph the way a model captures its layers.
    layers = 1
    if args.graph:
        layers = max(d for d in range(1, max(1, args.graph_layers) + 1) if args.steps % d == 0)
        for _ in range(3):
            eager_step()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(layers):
                eager_step()
        step = graph.replay

    def timed(fn, calls):
        a, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        a.record()
        for _ in range(calls):
            fn()
        e.record()
        torch.cuda.synchronize()
        return time.perf_counter() - t0, a.elapsed_time(e) * 1e-3

    clock_ramp(step)                                          # (before the W warm-up steps; untimed)
    for _ in range(-(-args.warmup // layers)):
        step()
    wall, dev_s = timed(step, args.steps // layers)
    us_per_step = wall / args.steps * 1e6
    dev_step_avg = dev_s / args.steps * 1e6

    # per-call brackets (an event pair around every call): the time of a call that starts on an idle queue, dispatch latency
    # included
    def event_time(fn, n):
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
        for a, e in ev:
            a.record()
            fn()
            e.record()
        torch.cuda.synchronize()
        ts = sorted(a.elapsed_time(e) * 1e3 for a, e in ev)
        return sum(ts) / len(ts), ts[len(ts) // 2]

    eager_wall, eager_dev = timed(eager_step, args.steps)
    eager_iso_avg, eager_iso_med = event_time(eager_step, args.steps)
    # the same step as a captured HIP graph, one step per graph, replayed args.steps times (the serving path runs whole
    # decode steps from graphs; beside the eager figure, never instead of it)
    one_graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(one_graph):
        eager_step()
    clock_ramp(one_graph.replay)                              # (the capture left the queue idle: same ramp as the eager figure gets)
    _, graph_dev = timed(one_graph.replay, args.steps)
    # the dominant kernel alone: args.steps launches queued back to back between one pair of events (the launches are
    # shorter on the host than on the GPU, so the queue never runs dry), and the per-launch brackets beside it
    split_only = lambda: K.decode(g["q_nope"], g["q_rope"], g["nope"], g["rope"], g["block_table"], g["seq_lens"],
                                  case["scale"], out_v, q_len=q_len, num_splits=splits, workspace=ws, phase="split")
    for _ in range(3):
        split_only()
    _, k_dev = timed(split_only, args.steps)
    k_back_to_back = k_dev / args.steps * 1e6
    k_iso_avg, k_med = event_time(split_only, args.steps)
    # ... and where it runs: args.steps whole steps queued as in the timed region above, the split phase of each bracketed
    # by its own pair of events (the two phases as two calls); this is the duration a kernel trace of this command shows
    reduce_only = lambda: K.decode(g["q_nope"], g["q_rope"], g["nope"], g["rope"], g["block_table"], g["seq_lens"],
                                   case["scale"], out_v, q_len=q_len, num_splits=splits, workspace=ws, phase="reduce")
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    for _ in range(args.warmup):
        eager_step()
    torch.cuda.synchronize()
    split_with_write = lambda: K.decode(g["q_nope"], g["q_rope"], g["nope"], g["rope"], g["block_table"], g["seq_lens"],
                                        case["scale"], out_v, q_len=q_len, num_splits=splits, workspace=ws, phase="split",
                                        new_rows=(g["new_c"], g["new_r"], g["slot_mapping"]))
    for a, e in ev:
        a.record()
        split_with_write()
        e.record()
        reduce_only()
    torch.cuda.synchronize()
    k_avg = sum(a.elapsed_time(e) for a, e in ev) / len(ev) * 1e3
    power = None if args.no_power_probe else socket_power(split_only)

    ab = algorithmic_bytes(case, heads)
    sum_l = int(case["seq_lens"].sum())
    flops = sum_l * heads * q_len * 2 * (576 + 512)
    kern_bytes = ab["kv"] + ab["q"] + ab["tables"]          # what the split kernel must read (partials excluded)
    achieved = kern_bytes / (k_avg * 1e-6) / 1e9
    # HBM bytes per launch of the split kernel from the FETCH_SIZE / WRITE_SIZE counter runs (scaled on a plain copy) of
    # exactly this workload; a counter run cannot be made from inside this script, so other shapes report null
    default_shape = (args.seed, b, args.len_lo, args.len_hi, q_len, splits) == (0, 64, 4096, 8192, 1, 4) and not args.l2_resident
    profile_of = {128: "mla_decode_v3_b64_ctx8k.md", 16: "mla_decode_v3_b64_ctx8k_16heads.md"}
    traffic, traffic_src = profile_traffic(profile_of.get(heads, ""), default_shape and heads in profile_of)
    row_groups = 1 if heads * q_len <= 32 else (2 if heads * q_len <= 64 else 4)   # the kernel form the library picks
    res = {
        "metric": f"MLA decode us/layer (B={b}, ctx {args.len_lo // 1024}k-{args.len_hi // 1024}k, {heads} heads, bf16, cache write + split-KV decode + reduce)",
        "value": round(dev_step_avg, 2), "unit": "us/layer", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(us_per_step / 1e3, 5), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "configs[1]: absorbed-MLA paged decode, DeepSeek-V3 shape", "batch": b, "heads": heads,
                   "q_len": q_len, "seq_lens": f"uniform[{args.len_lo},{args.len_hi}]", "sum_seq_len": sum_l,
                   "page": 128, "kv_splits": splits, "seed": args.seed},
        "step_us": {"host_wall": round(us_per_step, 2), "device_avg": round(dev_step_avg, 2),
                    "launch": f"hip graph replay, {layers} steps per graph" if args.graph else "eager launches, queued",
                    "eager_host_wall": round(eager_wall / args.steps * 1e6, 2),
                    "eager_device_queued": round(eager_dev / args.steps * 1e6, 2),
                    "hip_graph_replay": round(graph_dev / args.steps * 1e6, 2),
                    "eager_device_one_step_alone_avg": round(eager_iso_avg, 2),
                    "eager_device_one_step_alone_median": round(eager_iso_med, 2)},
        "step_tflops": round(flops / (dev_step_avg * 1e-6) / 1e12, 1),
        "step_hbm_gbs": round(ab["total"] / (dev_step_avg * 1e-6) / 1e9, 1),
        "step_roofline_frac": round(max(ab["total"] / (HBM_PEAK_GBS * 1e9), flops / (MFMA_BF16_PEAK_TFLOPS * 1e12))
                                    / (dev_step_avg * 1e-6), 4),
        "roofline": {"kernel": f"mla_decode_v3_kernel<false, false, {row_groups}, true>", "bound": "hbm", "achieved": round(achieved, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
                     "traffic_source": traffic_src,
                     "kernel_us_avg": round(k_avg, 2), "kernel_us_back_to_back_avg": round(k_back_to_back, 2),
                     "kernel_us_one_launch_alone_avg": round(k_iso_avg, 2),
                     "kernel_us_one_launch_alone_median": round(k_med, 2),
                     "algorithmic_bytes": kern_bytes, "kernel_tflops": round(flops / (k_avg * 1e-6) / 1e12, 1),
                     "mfma_frac": round(flops / (k_avg * 1e-6) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
                     "socket_power": power},
    }

    if not args.no_cpu_baseline:
        from oracle import mla_oracle as O
        cpu_info = cpu_fields()
        ns = min(args.cpu_seqs, b)
        sl = slice(0, ns * q_len)
        cn, cr = case["nope"].clone(), case["rope"].clone()      # the oracle sees the same new rows in its cache
        O.cache_write(cn, case["slot_mapping"], case["new_c"])
        O.cache_write(cr, case["slot_mapping"], case["new_r"])

        def cpu_once():
            return O.absorbed_decode(case["q_nope"][sl], case["q_rope"][sl], cn, cr,
                                     case["block_table"][:ns], case["seq_lens"][:ns], case["scale"])
        cpu_once()
        ts = []
        for _ in range(3):
            c0 = time.perf_counter()
            ref = cpu_once()
            ts.append(time.perf_counter() - c0)
        sample_l = int(case["seq_lens"][:ns].sum())
        cpu_us_full = sorted(ts)[1] * 1e6 * sum_l / sample_l
        err = (out_v[sl].float().cpu() - ref).abs()
        res["cpu_baseline"] = {"value": round(cpu_us_full, 1), "unit": "us/layer", **cpu_info, "kind": "port",
                               "sample": f"oracle (torch fp32) on the first {ns} of {b} sequences ({sample_l} of {sum_l} "
                                         f"cached tokens), median of 3, scaled by token count",
                               "sample_seconds": round(sorted(ts)[1], 3), "gpu_vs_oracle_max_abs": round(err.max().item(), 5)}
        res["gpu_vs_oracle"] = parity_fields(err, ref, "bf16", sequences=ns)
        res["parity_ok"] = res["gpu_vs_oracle"]["parity_ok"]
    if args.l2_resident:
        res["config"]["probe"] = "block table folded onto 8 pages: cache rows from L2, not the workload's HBM traffic"
    if args.gemm_probe:
        res["gemm_probe_tflops"] = gemm_probe(dev)
    default_run = (args.seed, b, heads, args.len_lo, args.len_hi, q_len) == (0, 64, 128, 4096, 8192, 1) and not args.l2_resident
    if default_run and not args.no_secondary:
        # the other single-GPU configurations, short: after the headline measurement and outside its timed region
        del g, out, out_v, ws
        torch.cuda.empty_cache()
        short = argparse.Namespace(**{**vars(args), "steps": 5, "warmup": 2, "no_power_probe": True})
        res["secondary"] = {}
        for name, fn in (("configs[2]", bench_prefill), ("configs[3]", bench_dsa), ("configs[4]", bench_fp8)):
            r = fn(K, dev, short)
            res["secondary"][name] = {k: r[k] for k in ("metric", "value", "unit", "gpu_vs_oracle", "parity_ok", "chain_us",
                                                        "step_us", "chain_roofline") if k in r}
            res["secondary"][name]["roofline"] = {k: r["roofline"][k] for k in ("kernel", "bound", "achieved", "peak", "unit", "frac")}
            del r
            torch.cuda.empty_cache()
    finish(res)


if __name__ == "__main__":
    main()

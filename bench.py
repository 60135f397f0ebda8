"""Benchmark of the structured-loss hot path on one MI355X.

A step is one training pass over one WMT14 En-De shaped batch (B=40, L=128, T=32, V=40000, fp16 logits):
logsoftmax_gather -> eos mask -> inside forward + backward -> loss -> logsoftmax_gather backward (in place), the work
autograd performs for the criterion.  Inputs are resident in HBM before the timed region; each step consumes a fresh
logits buffer because the path overwrites it with the gradient.

Prints one JSON line: whole-job throughput in sentences/s, the HBM roofline of the dominant kernel (the in-place
logsoftmax_gather backward: logits read, gradient written) from HIP events recorded around it inside the timed region,
and the CPU oracle timed on the host cores over a bounded sample of the same batch.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth
# Bytes per launch of the roofline kernel at this workload as the L2 caches request them from the memory side, from
# rocprofv3 FETCH_SIZE / WRITE_SIZE scaled against a plain device copy of known size; summary in
# profiles/lsg_cfg2_hbm_traffic_pmc.md.  None = not measured for this build.  (lsg_bwd: the single-call step at this
# batch's lengths - 3408 of 5120 rows read and written.  Part of its reads are served by the 256 MB memory-side cache, where
# the forward pass leaves the rows, which is how the kernel exceeds the rate of a device copy.)
EVENT_EVERY = 5  # steps between two bracketed launches of the roofline kernel inside the timed region
ROOFLINE_KERNEL = {"single": "lsg_bwd", "fused": "lsg_bwd", "unfused": "lsg_fwd"}
ROOFLINE_KERNEL_NAME = {"lsg_bwd": "lsg_bwd_kernel<half, from logits>", "lsg_fwd": "lsg_fwd_kernel<half, grad>"}
MEASURED_TRAFFIC_BYTES = {"lsg_bwd": 546.65e6, "lsg_fwd": 273.84e6}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--cpu-sentences", type=int, default=40, help="sentences of the batch timed on the CPU oracle")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-decode", action="store_true", help="skip the legs beyond the training step (same as --legs autograd,operator)")
    ap.add_argument("--legs", default="all",
                    help="comma-separated legs to run beside the headline step: autograd, operator, decode, glat, long, links, maxleft3, "
                         "frontend (default: all; 'none' for the headline alone) - for profiling runs that want few kernels")
    ap.add_argument("--decode-sentences", type=int, default=1000,
                    help="sentences of the inference configuration the decode leg uses (default: all 1000)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain device copy of a logits-sized fp16 buffer (409.6 MB read, 409.6 MB written): "
                         "the reference point for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE counters")
    ap.add_argument("--step", choices=["single", "fused"], default="single",
                    help="single: one native call per step (default); fused: four native calls from Python")
    ap.add_argument("--unfused", action="store_true",
                    help="issue the criterion's glue (eos mask, gradient scaling) as separate torch ops, like the reference")
    return ap.parse_args()


def cpu_baseline(batch_cpu, logits_sample, n_sent, budget_s=10.0, max_runs=200):
    """The oracle (a C port of the reference loops, OpenMP over rows / sentences) on the first n_sent sentences: runs of
    the whole training pass until about ``budget_s`` seconds of CPU work are spent (at least 9 runs), the median taken."""
    import numpy as np
    import torch
    from oracle import oracle
    from pcfg_nat_amd import harness

    ol = batch_cpu["output_length"][:n_sent]
    tl = batch_cpu["target_length"][:n_sent]
    links = batch_cpu["links"][:n_sent].numpy()
    targets = batch_cpu["targets"][:n_sent]
    L = links.shape[1]
    idx = targets.unsqueeze(1).expand(-1, L, -1).numpy()
    x = logits_sample.float().numpy()
    times = []
    t_begin = time.perf_counter()
    while len(times) < 10 or (time.perf_counter() - t_begin < budget_s and len(times) <= max_runs):
        t0 = time.perf_counter()
        sel, probs = oracle.lsg_fwd(x, idx, want_probs=True, dtype=np.float32)
        match = harness.eos_masked(torch.from_numpy(sel), ol, tl).numpy()
        S, C = oracle.inside_fwd(match, links, ol.numpy(), tl.numpy(), dtype=np.float32)
        mg, lg = oracle.inside_bwd(np.ones(n_sent, dtype=np.float32), S, C, match, links, ol.numpy(), tl.numpy(),
                                   dtype=np.float32)
        coef = (-1.0 / (tl.numpy() * n_sent)).astype(np.float32)
        oracle.lsg_bwd(probs, idx, mg * coef[:, None, None], dtype=np.float32)
        times.append(time.perf_counter() - t0)
    best = sorted(times[1:])[len(times[1:]) // 2]
    return {"value": n_sent / best, "unit": "sentences/s", "cores": oracle.num_threads(), "kind": "port",
            "sample": "first %d sentences of the same batch, fp32 oracle (logsoftmax_gather fwd+bwd, inside fwd+bwd), "
                      "median of %d runs after one warm-up, %.2f s per run" % (n_sent, len(times) - 1, best)}


def _percentile(sorted_vals, q):
    return sorted_vals[min(len(sorted_vals) - 1, int(q * len(sorted_vals)))]


def cpu_model_string():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def _cpu_viterbi_decode(ob, tok, links, m, mask):
    """The oracle's Viterbi decode of one batch on the host (pcfg_viterbi.cu:22-140 and pcfg_loss.cpp:12-73 restated in C,
    OpenMP over the sentences; the length selection of glat_decomposed_with_link_two_hands_tri_pcfg.py:489-497 in numpy).
    Returns (seconds, tokens float32 [B,maxlen], pred_length [B])."""
    import numpy as np
    from oracle import oracle
    from pcfg_nat_amd import synth

    t0 = time.perf_counter()
    S, R, Lt, M = oracle.viterbi(ob, links, m, dtype=np.float32)
    Lq = S.shape[2]
    with np.errstate(divide="ignore", invalid="ignore"):
        sc = S[:, 1, :] / np.arange(Lq, dtype=np.float32)[None, :]
    sc = np.where(np.isnan(sc), -np.inf, sc)
    pred = sc[:, 1:].argmax(-1) + 1
    out = oracle.viterbi_decoding(pred, m, Lt, R, M, tok, mask, synth.PAD)
    return time.perf_counter() - t0, out, pred


def decode_timing(dev, cpu=True, front_end_sample=16, n_sent=1000):
    """Viterbi decode of the inference configuration (BASELINE config 4: 1000 sentences, src ~U[5,100], L = 4*src, V=40000,
    fp16 logits ~N(0,3)) as the model runs it: front-end (log-softmax + max over the vocabulary, one read of the logits)
    followed by tables + length selection + readout, all enqueued by one native call; the emitted token counts are read back
    by the host, which is the decode's one synchronisation.  Batch 1: wall-clock latency of every one of the 1000 sentences
    (median, 95th percentile, mean; front-end and decode also timed apart).  Batch 64: throughput over all 16 length-sorted
    batches of the same 1000 sentences (15 of 64 and one of 40).  With ``cpu`` the same sentences are decoded by the oracle
    on the host cores from the node scores the GPU front-end produced (batch 1: one sentence, hence one core, at a time;
    batch 64: OpenMP over the sentences), the front-end by torch's CPU ``log_softmax`` + ``max`` on a strided sample of
    ``front_end_sample`` sentences; the tokens of both paths are compared."""
    import numpy as np
    import torch
    from pcfg_nat_amd import custom_ops as ops, harness, synth

    V = 40000
    lens = synth.config4_lengths()[:n_sent]
    n_sent = len(lens)
    out = {"sentences": n_sent,
           "src_length_histogram": {"%d-%d" % (lo, lo + 19): int(((lens >= lo) & (lens < lo + 20)).sum()) for lo in range(5, 101, 20)}}
    gen = torch.Generator().manual_seed(3)
    ggen = torch.Generator(device=dev).manual_seed(4)

    def make(src):
        m = 4 * src
        L = int(m.max())
        links = synth.make_links(len(src), L, m, 1, gen)
        logits = (torch.randn(len(src), L, V, device=dev, dtype=torch.float32, generator=ggen) * 3).half()
        mask = synth.support_masks(L, 1)[0]
        return {"logits": logits, "links": links.to(dev), "m": m.to(dev), "mask": mask.to(dev),
                "links_cpu": links.numpy() if cpu else None, "m_cpu": m.numpy(), "mask_cpu": mask.numpy()}

    def run(c):
        return harness.decode_from_logits(c["logits"], c["links"], c["m"], c["mask"], single_call=True)

    def wall(fn):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        res = fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3, res

    def cpu_front_end(cases):
        """torch on the host cores: log_softmax over the vocabulary and max, per sampled sentence; ms per graph node."""
        ms = nodes = 0
        for c in cases:
            x = c["logits"].cpu()
            t0 = time.perf_counter()
            torch.log_softmax(x.float(), dim=-1).max(dim=-1)
            ms += (time.perf_counter() - t0) * 1e3
            nodes += x.shape[0] * x.shape[1]
        return ms / nodes

    try:
        cases = [make(lens[i:i + 1]) for i in range(n_sent)]
        for c in cases:  # one untimed pass: every kernel variant the lengths select has been loaded once
            run(c)
        timed = [wall(lambda c=c: run(c)) for c in cases]
        total = sorted(t for t, _ in timed)
        front = sorted(wall(lambda c=c: ops.logsoftmax_max(c["logits"]))[0] for c in cases)
        pre = [ops.logsoftmax_max(c["logits"]) for c in cases]
        dec = sorted(wall(lambda c=c, o=o: harness.viterbi_decode(o[0], o[1], c["links"], c["m"], c["mask"], single_call=True))[0]
                     for c, o in zip(cases, pre))
        out["b1"] = {"sentences": len(cases),
                     "ms_per_sentence_p50": _percentile(total, 0.5), "ms_per_sentence_p95": _percentile(total, 0.95),
                     "ms_per_sentence_mean": sum(total) / len(total),
                     "front_end_ms_p50": _percentile(front, 0.5), "front_end_ms_p95": _percentile(front, 0.95),
                     "decode_ms_p50": _percentile(dec, 0.5), "decode_ms_p95": _percentile(dec, 0.95),
                     "decode_ms_mean": sum(dec) / len(dec)}
        out["b1_ms_per_sentence"] = out["b1"]["ms_per_sentence_p50"]
        out["host_polling_still_on"] = bool(ops._pinned_counts.polling_on())
        if cpu:
            from oracle import oracle
            per, same = [], True
            for c, o, (_, got) in zip(cases, pre, timed):
                sec, want, want_len = _cpu_viterbi_decode(o[0].cpu().numpy(), o[1].cpu().numpy(), c["links_cpu"], c["m_cpu"], c["mask_cpu"])
                per.append(sec * 1e3)
                same = same and np.array_equal(got[0].cpu().numpy(), want) and np.array_equal(got[1].cpu().numpy(), want_len)
            per.sort()
            fe = cpu_front_end(cases[::max(1, n_sent // front_end_sample)][:front_end_sample])
            mean_nodes = float(4 * lens.double().mean())
            out["cpu_b1"] = {"kind": "port", "cores": 1, "threads_available": oracle.num_threads(), "sentences": len(per),
                             "decode_ms_p50": _percentile(per, 0.5), "decode_ms_p95": _percentile(per, 0.95),
                             "decode_ms_mean": sum(per) / len(per),
                             "front_end_ms_per_node": fe, "front_end_ms_mean_sentence": fe * mean_nodes,
                             "front_end_sample": "%d sentences, every %d-th of the 1000, torch CPU log_softmax(float32) + max on %d threads"
                                                 % (front_end_sample, max(1, n_sent // front_end_sample), torch.get_num_threads()),
                             "ms_per_sentence_mean": sum(per) / len(per) + fe * mean_nodes,
                             "tokens_equal_gpu": bool(same)}
        del cases, pre, timed
        # batch 64: all sentences, sorted by length
        srt = torch.sort(lens)[0]
        chunks = [make(srt[i:i + 64]) for i in range(0, n_sent, 64)]
        for c in chunks:  # untimed pass, as above
            run(c)
        t_all, got = wall(lambda: [run(c) for c in chunks])
        pre = [ops.logsoftmax_max(c["logits"]) for c in chunks]
        t_dec, _ = wall(lambda: [harness.viterbi_decode(o[0], o[1], c["links"], c["m"], c["mask"], single_call=True) for c, o in zip(chunks, pre)])
        out["b64_batches"] = len(chunks)
        out["b64_sentences_per_s"] = n_sent / (t_all * 1e-3)
        out["b64_decode_only_sentences_per_s"] = n_sent / (t_dec * 1e-3)
        if cpu:
            sec, same = 0.0, True
            for c, o, g in zip(chunks, pre, got):
                s1, want, want_len = _cpu_viterbi_decode(o[0].cpu().numpy(), o[1].cpu().numpy(), c["links_cpu"], c["m_cpu"], c["mask_cpu"])
                sec += s1
                same = same and np.array_equal(g[0].cpu().numpy(), want) and np.array_equal(g[1].cpu().numpy(), want_len)
            nodes = float(sum(c["logits"].shape[0] * c["logits"].shape[1] for c in chunks))
            out["cpu_b64"] = {"kind": "port", "cores": oracle.num_threads(), "decode_only_sentences_per_s": n_sent / sec,
                              "sentences_per_s_with_front_end": n_sent / (sec + out["cpu_b1"]["front_end_ms_per_node"] * nodes * 1e-3),
                              "tokens_equal_gpu": bool(same)}
    except RuntimeError as e:  # a shape the library does not build yet
        out["error"] = str(e)[:200]
    return out


def glat_timing(logits, targets, links, out_len, cpu=None):
    """The GLAT alignment pass that precedes the loss in every training step (nat_pcfg_loss.py:193-269) on the same
    batch, as one native call: gather + eos mask + arg max, inside forward, best tree, glancing glue.  ``cpu``: the CPU
    copies of (targets, links, output_length, target_length); the same pass is then also timed over the oracle on the host
    cores (torch CPU arg max, the oracle's gather, inside forward and best tree, the criterion's glue as torch CPU ops)."""
    import torch
    from pcfg_nat_amd import harness, synth

    B, L, _ = logits.shape
    prev = torch.full((B, L), 3, dtype=torch.int64, device=logits.device)
    prev = prev.masked_fill(torch.arange(L, device=logits.device).view(1, L) >= out_len.view(B, 1), synth.PAD)
    for _ in range(3):
        harness.glat_alignment(logits, targets, prev, links, 0.5, single_call=True)
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    reps = 20
    for _ in range(reps):
        harness.glat_alignment(logits, targets, prev, links, 0.5, single_call=True)
    end.record()
    torch.cuda.synchronize()
    res = {"ms_per_call": start.elapsed_time(end) / reps}
    if cpu is not None:
        import numpy as np
        from oracle import oracle

        tg, lk, ol, tl = cpu
        x = logits.cpu()
        prev_c = prev.cpu()

        class OracleOps:  # the two operators of the pass over the oracle, float32
            @staticmethod
            def dag_logsoftmax_gather_inplace(word_ins_out, select_idx):
                sel, _ = oracle.lsg_fwd(word_ins_out.numpy(), select_idx.numpy(), want_probs=False, dtype=np.float32)
                return word_ins_out, torch.from_numpy(sel)

            @staticmethod
            def cuda_pcfg_best_tree(match_all, links, output_length, target_length):
                m, k, o, t = match_all.numpy(), links.numpy(), output_length.numpy(), target_length.numpy()
                S, C = oracle.inside_fwd(m, k, o, t, dtype=np.float32)
                tree = oracle.best_tree(S, C, m, k, o, t, dtype=np.float32)
                return torch.from_numpy(tree), torch.from_numpy(S[:, 0, 0].copy())

        times = []
        for _ in range(4):
            t0 = time.perf_counter()
            harness.glat_alignment(x.float(), tg, prev_c, lk, 0.5, ops=OracleOps)
            times.append(time.perf_counter() - t0)
        best = sorted(times[1:])[1]
        res["cpu"] = {"kind": "port", "cores": oracle.num_threads(), "ms_per_call": best * 1e3,
                      "sample": "the same batch of %d sentences, float32 oracle + torch CPU glue, median of 3 runs after one warm-up" % B}
        res["speedup_vs_cpu"] = best * 1e3 / res["ms_per_call"]
    return res


def operator_api_timing(bufs, targets, links, ol, tl, args, timed_windows, host_enqueue_ms):
    """One training pass through the five drop-in names, driven by the criterion's own code under autograd
    (``harness.compute_pcfg_loss`` restates nat_pcfg_loss.py:98-145 call for call) and ``loss.backward()``; with a loss
    scale of 128 on top, as under ``--fp16``.  The logits reach the criterion as the non-leaf output of an upstream layer,
    which is played by a Function that hands out its buffer and swallows the gradient (no extra pass over the logits).

    The host's share is split three ways: the whole step; the two operators alone under autograd, fed with precomputed
    tensors in place of the criterion's glue (their wrappers, the autograd bookkeeping and the kernels); the four native
    calls behind them issued from Python without autograd."""
    import torch
    from pcfg_nat_amd import custom_ops as ops, harness, synth

    class UpstreamLayer(torch.autograd.Function):
        @staticmethod
        def forward(ctx, weight, buf):
            out = buf.new_empty(0)
            out.set_(buf.untyped_storage(), buf.storage_offset(), buf.shape, buf.stride())
            return out

        @staticmethod
        def backward(ctx, grad):
            return None, None

    B, L, _ = bufs[0].shape
    dev = bufs[0].device
    weight = torch.ones(1, device=dev, requires_grad=True)
    out_mask = torch.arange(L, device=dev).view(1, L) < ol.view(B, 1)
    tgt_mask = targets.ne(synth.PAD)

    def step(i, scale):
        lk = links.detach().requires_grad_(True)
        res = harness.compute_pcfg_loss(UpstreamLayer.apply(weight, bufs[i]), out_mask, targets, tgt_mask, lk)
        (res["loss"] * scale).backward()

    for i in range(args.warmup):
        step(i, 1.0)
    res = timed_windows(lambda i: step(i, 1.0))
    res["sentences_per_s_median"] = B / (res["ms_per_step_median"] * 1e-3)
    scaled = timed_windows(lambda i: step(i, 128.0), windows=3)
    res["loss_scale_128_ms_per_step_median"] = scaled["ms_per_step_median"]
    # These figures are bound by the host: the criterion's glue is some forty small torch kernels per step, and the host
    # takes as long to enqueue a step as the step takes on the wall clock.
    res["host_enqueue_ms_per_step"] = host_enqueue_ms(lambda i: step(i, 128.0))

    # the two operators alone, under autograd, the glue replaced by tensors computed once
    idx = targets.unsqueeze(1).expand(-1, L, -1)
    with torch.no_grad():
        _, m0 = ops.dag_logsoftmax_gather_inplace(bufs[0].clone(), idx)
        match_pre = harness.eos_masked(m0, ol, tl)
        w_pre = (-1.0 / (tl * B)).float() * 128.0
        g_pre = torch.zeros_like(match_pre)

    def operators_only(i):
        lk = links.detach().requires_grad_(True)
        ma = match_pre.detach().requires_grad_(True)
        _, sel = ops.dag_logsoftmax_gather_inplace(UpstreamLayer.apply(weight, bufs[i]), idx)
        ll = ops.cuda_pcfg_loss(ma, lk, ol, tl)
        ll.backward(w_pre)
        sel.backward(g_pre)

    for i in range(args.warmup):
        operators_only(i)
    res["operators_only_host_enqueue_ms_per_step"] = host_enqueue_ms(operators_only)
    res["operators_only_ms_per_step_median"] = timed_windows(operators_only, windows=3)["ms_per_step_median"]

    def native_calls_only(i):
        harness.train_step_fused(bufs[i], targets, links, ol, tl)

    for i in range(args.warmup):
        native_calls_only(i)
    res["four_native_calls_host_enqueue_ms_per_step"] = host_enqueue_ms(native_calls_only)
    res["glue_host_enqueue_ms_per_step"] = res["host_enqueue_ms_per_step"] - res["operators_only_host_enqueue_ms_per_step"]
    return res


def criterion_autograd_timing(bufs, targets, links, ol, tl, args, timed_windows, host_enqueue_ms):
    """The single call as a trainer adopts it: ``custom_ops.pcfg_criterion`` under autograd (one native call in the forward,
    one in the backward) followed by ``(loss * 128).backward()``, the logits arriving as the output of an upstream layer."""
    import torch
    from pcfg_nat_amd import custom_ops as ops

    class UpstreamLayer(torch.autograd.Function):
        @staticmethod
        def forward(ctx, weight, buf):
            out = buf.new_empty(0)
            out.set_(buf.untyped_storage(), buf.storage_offset(), buf.shape, buf.stride())
            return out

        @staticmethod
        def backward(ctx, grad):
            return None, None

    B = bufs[0].shape[0]
    weight = torch.ones(1, device=bufs[0].device, requires_grad=True)

    def step(i):
        lk = links.detach().requires_grad_(True)
        loss, _, _ = ops.pcfg_criterion(UpstreamLayer.apply(weight, bufs[i]), targets, lk, ol, tl)
        (loss * 128.0).backward()

    for i in range(args.warmup):
        step(i)
    res = timed_windows(step)
    res["sentences_per_s_median"] = B / (res["ms_per_step_median"] * 1e-3)
    res["host_enqueue_ms_per_step"] = host_enqueue_ms(step)
    res["loss_scale"] = 128.0
    return res


def long_sentence_timing(dev):
    """The single-call training pass at the long-sentence configuration (BASELINE config 3: B=8, L=512, T=140, V=40000,
    every sentence at full length), where the inside sweeps run their streaming kernels (256 main-chain nodes per
    sentence, link rows re-read from L2 every target position, one CU per sentence)."""
    import torch
    from pcfg_nat_amd import harness, synth

    B, L, T, V = 8, 512, 140, 40000
    gen = torch.Generator().manual_seed(2)
    m, n = torch.full((B,), L, dtype=torch.int64), torch.full((B,), T, dtype=torch.int64)
    links = synth.make_links(B, L, m, 1, gen).to(dev)
    targets = synth.make_targets(B, T, n, V, gen).to(dev)
    ol, tl = m.to(dev), n.to(dev)
    ggen = torch.Generator(device=dev).manual_seed(12)
    warm, reps = 2, 6
    bufs = [(torch.randn(B, L, V, device=dev, dtype=torch.float32, generator=ggen) * 2).half() for _ in range(warm + reps)]
    for i in range(warm):
        harness.train_step_single_call(bufs[i], targets, links, ol, tl)
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for i in range(warm, warm + reps):
        out = harness.train_step_single_call(bufs[i], targets, links, ol, tl)
    end.record()
    torch.cuda.synchronize()
    ms = start.elapsed_time(end) / reps
    return {"ms_per_step": ms, "sentences_per_s": B / (ms * 1e-3), "workload": "B=8, L=512, T=140, V=40000, fp16 logits"}


def link_scorer_timing(dev):
    """The model's link scorer after its projections at the training shape (B=40, L=128, 8 heads of 64, fp16 chunks):
    forward alone (what the glancing pass and inference run) and forward + backward."""
    import torch
    from pcfg_nat_amd import custom_ops as ops, synth

    B, L, H, F = 40, 128, 8, 64
    g = torch.Generator().manual_seed(0)
    q, kl, kr = ((torch.randn(B, L, H, F, generator=g) * 0.5).half().to(dev) for _ in range(3))
    gate = torch.randn(B, L, H, generator=g).half().to(dev)
    m, _ = synth._wmt_lengths(B, torch.Generator().manual_seed(1001), 10, L // 4, 32)
    prev = torch.full((B, L), 3).masked_fill(torch.arange(L).view(1, L) >= m.view(B, 1), synth.PAD).to(dev)
    lm, rm, mc = (x.to(dev) for x in synth.support_masks(L, 1))
    G = torch.randn(B, L, 2, L, generator=g).to(dev)

    def fwd():
        with torch.no_grad():
            return ops.pcfg_extract_links(q, kl, kr, gate, prev, synth.PAD, lm, rm, mc)

    G = G.masked_fill(~torch.isfinite(fwd()), 0)  # the upstream gradient of masked links is zero

    def fwd_bwd(products_inside=True):
        ts = [t.detach().requires_grad_(True) for t in (q, kl, kr, gate)]
        ops.pcfg_extract_links(*ts, prev, synth.PAD, lm, rm, mc, products_inside).backward(G)

    res = {}
    for name, fn in (("forward_ms", fwd), ("forward_backward_ms", fwd_bwd),
                     ("forward_backward_products_through_torch_ms", lambda: fwd_bwd(False))):
        for _ in range(10):
            fn()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        start.record()
        for _ in range(20):
            fn()
        end.record()
        torch.cuda.synchronize()
        res[name] = start.elapsed_time(end) / 20
    return res


def max_left3_timing(dev):
    """The inside loss forward + backward for ``--left-tree-layer 2`` (max_left = 3: a left subtree of up to three nodes
    under every main-chain node) at the training shape: B=40, L=130 (32 groups of four nodes), T=32, through
    ``cuda_pcfg_loss`` (forward with the eager backward inside, pcfg_loss.py:67-73)."""
    import torch
    from pcfg_nat_amd import custom_ops as ops, synth

    B, L, T, ml = 40, 130, 32, 3
    gen = torch.Generator().manual_seed(1003)
    src, n = synth._wmt_lengths(B, gen, 10, 32, T)  # src here = 4 * source length
    m = src + 2                                      # full groups: (m - 2) % (ml + 1) == 0
    links = synth.make_links(B, L, m, ml, gen).to(dev)
    match_all = torch.log_softmax(torch.randn(B, L, T, generator=gen) * 2, dim=-1).to(dev)
    ol, tl = m.to(dev), n.to(dev)

    def step():
        ma = match_all.detach().requires_grad_(True)
        lk = links.detach().requires_grad_(True)
        return ops.cuda_pcfg_loss(ma, lk, ol, tl)

    def timed(reps):
        for _ in range(3):
            step()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        start.record()
        for _ in range(reps):
            ll = step()
        end.record()
        torch.cuda.synchronize()
        return start.elapsed_time(end) / reps, ll

    ms, ll = timed(20)
    res = {"ms_per_call": ms, "sentences_per_s": B / (ms * 1e-3), "valid_sentences": int(torch.isfinite(ll).sum()),
           "path": ops.max_left_path(ml, L, T), "workload": "B=40, L=130, T=32, max_left=3, inside forward + backward"}
    was = ops.max_left3_tuned(0)  # the same call through the plain one-workgroup-per-sentence kernels
    try:
        ms_plain, ll_plain = timed(5)
    finally:
        ops.max_left3_tuned(was)
    res["plain_kernels_ms_per_call"] = ms_plain
    res["speedup_vs_plain_kernels"] = ms_plain / ms
    res["log_likelihoods_agree"] = bool(torch.allclose(ll, ll_plain, rtol=1e-5))
    res["viterbi_decode"] = max_left3_decode_timing(dev)
    return res


def max_left3_decode_timing(dev):
    """The single-call Viterbi decode (tables, length selection, walk) for ``--left-tree-layer 2`` on graphs of 130, 258 and
    402 nodes (source lengths 32, 64, 100) at batch 1 and of 258 nodes at batch 64, wall clock per call, with the
    one-launch table kernel and with the plain kernel."""
    import time
    import torch
    from pcfg_nat_amd import custom_ops as ops, synth

    ml, out = 3, []
    gen = torch.Generator().manual_seed(1004)
    for B, L in ((1, 130), (1, 258), (1, 402), (64, 258)):
        m = torch.full((B,), L, dtype=torch.int64)
        links = synth.make_links(B, L, m, ml, gen).to(dev)
        ob, tok = synth.ob_and_tokens(torch.randn(B, L, 48, generator=gen) * 3)
        mask = synth.support_masks(L, ml)[0].to(dev)
        args = (ob.to(dev), links, m.to(dev), tok.to(dev), mask, synth.PAD)

        def timed(reps):
            for _ in range(2):
                ops.pcfg_viterbi_decode(*args)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(reps):
                got = ops.pcfg_viterbi_decode(*args)
            torch.cuda.synchronize()
            return (time.perf_counter() - t0) / reps * 1e3, got

        ms, got = timed(20)
        was = ops.max_left3_tuned(0)
        try:
            ms_plain, got_plain = timed(3)
        finally:
            ops.max_left3_tuned(was)
        out.append({"batch": B, "graph_nodes": L, "ms_per_call": ms, "plain_kernel_ms_per_call": ms_plain,
                    "speedup_vs_plain_kernel": ms_plain / ms, "emitted_tokens_max": int(got[0].size(1)),
                    "same_tokens": bool(torch.equal(got[0], got_plain[0]) and torch.equal(got[1], got_plain[1]))})
    return out


def decode_front_end_timing(dev):
    """max_v log_softmax and arg max over the vocabulary in one read of the logits (the model's decode front-end) at
    B=64, L=400, V=40000 fp16 (2.05 GB)."""
    import torch
    from pcfg_nat_amd import custom_ops as ops

    B, L, V = 64, 400, 40000
    ggen = torch.Generator(device=dev).manual_seed(13)
    x = (torch.randn(B, L, V, device=dev, dtype=torch.float32, generator=ggen) * 3).half()
    for _ in range(2):
        ops.logsoftmax_max(x)
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(5):
        ops.logsoftmax_max(x)
    end.record()
    torch.cuda.synchronize()
    ms = start.elapsed_time(end) / 5
    nbytes = B * L * V * 2 + B * L * 12
    return {"ms_per_call": ms, "gb_per_s": nbytes / (ms * 1e-3) / 1e9, "workload": "B=64, L=400, V=40000, fp16 logits"}


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this path runs on one GPU (sentences are independent; nothing here uses a second device); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    from pcfg_nat_amd import harness, synth, _lib

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    _lib.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    B, L, T, V = 40, 128, 32, 40000
    gen = torch.Generator().manual_seed(1001)
    m, n = synth._wmt_lengths(B, gen, 10, L // 4, T)
    g2 = torch.Generator().manual_seed(1)
    links_cpu = synth.make_links(B, L, m, 1, g2)
    targets_cpu = synth.make_targets(B, T, n, V, g2)
    links, targets = links_cpu.to(dev), targets_cpu.to(dev)
    ol, tl = m.to(dev), n.to(dev)

    total = args.steps + args.warmup
    ggen = torch.Generator(device=dev).manual_seed(11)
    bufs = [(torch.randn(B, L, V, device=dev, dtype=torch.float32, generator=ggen) * 2).half() for _ in range(total)]
    sample_logits = bufs[args.warmup][:args.cpu_sentences].cpu() if not args.no_cpu_baseline else None
    torch.cuda.synchronize()

    if args.calibrate_copy:
        dst = torch.empty_like(bufs[0])
        dst.copy_(bufs[0])
        torch.cuda.synchronize()
        del dst
    pairs = {}

    detail = {"on": False}  # timed region: events around the roofline kernel only; afterwards: around all four
    mode = "unfused" if args.unfused else args.step
    roof = ROOFLINE_KERNEL[mode]

    sampled = {"step": 0}
    pool = []

    def mark(name, phase):
        if name == "events":  # single-call step: the library records the events we hand out around its kernels
            # Inside the timed region the roofline kernel is bracketed in every fifth step only: a pair of timing events
            # holds up the queue by about 20 us, a tenth of the step.  The events of the region are created and
            # materialised ahead of it (the pool), so that the region holds only the two records around the kernel.
            sampled["step"] += 1
            if not detail["on"] and (sampled["step"] - 1) % EVENT_EVERY != 0:
                return None
            evs = []
            for kernel in ("lsg_fwd", "inside_fwd_bwd", "lsg_bwd"):
                for _ in range(2):
                    if kernel != roof and not detail["on"]:
                        evs.append(None)
                        continue
                    if pool:
                        ev = pool.pop()
                    else:
                        ev = torch.cuda.Event(enable_timing=True)
                        ev.record()  # materialises the HIP event; the library records it again at the right place
                    pairs.setdefault(kernel, []).append(ev)
                    evs.append(ev)
            return evs
        if name != roof and not detail["on"]:
            return
        ev = torch.cuda.Event(enable_timing=True)
        ev.record()
        pairs.setdefault(name, []).append(ev)

    step_fn = {"unfused": harness.train_step_direct, "fused": harness.train_step_fused, "single": harness.train_step_single_call}[mode]
    B_timed = B  # sentences whose logsoftmax_gather launch the timing events bracket
    losses = []
    for i in range(args.warmup):
        losses.append(step_fn(bufs[i], targets, links, ol, tl)[0])
    if mode == "single":
        for _ in range(2 * ((args.steps + EVENT_EVERY - 1) // EVENT_EVERY)):
            ev = torch.cuda.Event(enable_timing=True)
            ev.record()
            pool.append(ev)
    torch.cuda.synchronize()
    sampled["step"] = 0
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for i in range(args.warmup, total):
        losses.append(step_fn(bufs[i], targets, links, ol, tl, mark=mark)[0])
    end.record()
    torch.cuda.synchronize()
    ms = start.elapsed_time(end) / args.steps
    assert all(torch.isfinite(x) for x in losses), "non-finite loss"

    def averages():
        out = {}
        for name, evs in pairs.items():
            d = [evs[2 * i].elapsed_time(evs[2 * i + 1]) for i in range(len(evs) // 2)]
            out[name] = sum(d) / len(d)
        return out

    def fresh_logits():
        for i in range(args.warmup, total):  # the path has overwritten the buffers with gradients
            bufs[i].copy_(torch.randn(B, L, V, device=dev, dtype=torch.float32, generator=ggen).mul_(2))

    def host_enqueue_ms(fn):
        """Host time to enqueue one step of ``fn`` (no wait for the GPU inside the window)."""
        fresh_logits()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(args.warmup, total):
            fn(i)
        t1 = time.perf_counter()
        torch.cuda.synchronize()
        return (t1 - t0) * 1e3 / args.steps

    def timed_windows(fn, windows=5):
        """ms per step of ``fn(i)`` over several windows of args.steps steps each; every window gets fresh logits."""
        per = []
        for _ in range(windows):
            fresh_logits()
            s0, s1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            s0.record()
            for i in range(args.warmup, total):
                fn(i)
            s1.record()
            torch.cuda.synchronize()
            per.append(s0.elapsed_time(s1) / args.steps)
        per.sort()
        return {"windows": windows, "steps_per_window": args.steps, "ms_per_step_median": per[len(per) // 2],
                "ms_per_step_min": per[0], "ms_per_step_max": per[-1]}

    kern_ms = averages()  # the roofline kernel only: measured inside the timed region
    roof_launches = len(pairs[roof]) // 2
    # per-kernel detail from a separate instrumented pass over buffers that have already been consumed (same work:
    # every value is finite, the kernels do not branch on data)
    roof_in_region = kern_ms[roof]
    pairs.clear()
    detail["on"] = True
    for i in range(min(5, total)):
        step_fn(bufs[i], targets, links, ol, tl, mark=mark)
    torch.cuda.synchronize()
    kern_ms = averages()
    kern_ms[roof] = roof_in_region
    # the single-call step neither reads the logits of the pad nodes behind a sentence's graph nor re-reads them in the
    # backward (their gradient rows are written as zeros); the other modes go through the operator API, which cannot know
    live_rows = int(m[:B_timed].sum()) if mode == "single" else None
    fwd_bytes = synth.lsg_fwd_bytes(B_timed, L, V, T, 2, require_grad=(mode == "unfused"), live_rows=live_rows)
    # (at this graph size the zeros of the pad rows are written by the launch that holds the sweeps, not by the backward)
    bwd_bytes = synth.lsg_bwd_bytes(B_timed, L, V, T, 2, live_rows=live_rows, pads_zeroed_elsewhere=(mode == "single"))
    roof_bytes = bwd_bytes if roof == "lsg_bwd" else fwd_bytes
    achieved = roof_bytes / (kern_ms[roof] * 1e-3) / 1e9
    traffic = MEASURED_TRAFFIC_BYTES[roof]

    result = {
        "metric": "inside fwd+bwd sentences/s at B=40,L=128,T=32,V=40k; Viterbi ms/sentence",
        "value": B / (ms * 1e-3),
        "unit": "sentences/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16 logits, f32 arithmetic",
        "data": "synthetic",
        "config": {"workload": "WMT14 En-De shaped training batch (BASELINE config 2): B=40, L=128, T=32, V=40000, "
                               "fp16 logits ~N(0,2), src ~U[10,32] x4, max_left=1; logsoftmax_gather fwd -> eos mask -> "
                               "inside fwd+bwd -> loss -> logsoftmax_gather bwd (%s); criterion glue "
                               % ("forward overwrites the logits with softmax, four passes over the logits" if mode == "unfused"
                                  else "forward read-only, backward recomputes softmax from row log-sum-exps, three passes "
                                       "over the logits")
                               + ("as separate torch ops" if args.unfused else "folded into the kernels, %s" %
                                  ("one native call per step" if args.step == "single" else "four native calls per step")),
                   "global_batch": B, "graph_nodes": L, "target_len": T, "vocab": V},
        "roofline": {"bound": "hbm", "kernel": ROOFLINE_KERNEL_NAME[roof], "achieved": achieved, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                     "traffic": (traffic * B_timed / B) if traffic else None,
                     "algorithmic_bytes": roof_bytes, "avg_ms": kern_ms[roof], "launches_timed": roof_launches,
                     "sentences_per_launch": B_timed,
                     "rows_per_launch": B_timed * L, "rows_read": live_rows if live_rows is not None else B_timed * L},
        "kernels_ms": kern_ms,
        "lsg_fwd_gbs": fwd_bytes / (kern_ms["lsg_fwd"] * 1e-3) / 1e9,
        "lsg_bwd_gbs": bwd_bytes / (kern_ms["lsg_bwd"] * 1e-3) / 1e9,
    }
    # the same step over several windows (the headline above is one window of args.steps steps)
    result["headline_windows"] = timed_windows(lambda i: step_fn(bufs[i], targets, links, ol, tl))
    result["headline_windows"]["sentences_per_s_median"] = B / (result["headline_windows"]["ms_per_step_median"] * 1e-3)
    if mode == "single":
        # the same single call with an upstream factor of 128 on the loss (fp16 loss scaling), folded into the weights
        sc = timed_windows(lambda i: harness.train_step_single_call(bufs[i], targets, links, ol, tl, loss_scale=128.0))
        sc["sentences_per_s_median"] = B / (sc["ms_per_step_median"] * 1e-3)
        sc["loss_scale"] = 128.0
        result["single_call_scaled"] = sc
    # the drop-in path: the unchanged criterion code over the operator API under autograd (dag_logsoftmax_gather_inplace ->
    # eos mask -> cuda_pcfg_loss -> loss -> backward), which reads and rewrites every row (it is not told the lengths)
    legs = {"autograd", "operator", "decode", "glat", "long", "links", "frontend", "maxleft3"}
    if args.legs != "all":
        legs = {x for x in args.legs.split(",") if x and x != "none"}
    if args.no_decode:
        legs &= {"autograd", "operator"}
    from pcfg_nat_amd import custom_ops
    result["host_backend"] = custom_ops.host_backend()
    if "autograd" in legs:
        result["criterion_autograd"] = criterion_autograd_timing(bufs, targets, links, ol, tl, args, timed_windows, host_enqueue_ms)
    if "operator" in legs:
        result["operator_api"] = operator_api_timing(bufs, targets, links, ol, tl, args, timed_windows, host_enqueue_ms)
    cpu = not args.no_cpu_baseline
    if "decode" in legs:
        result["viterbi"] = decode_timing(dev, cpu=cpu, n_sent=args.decode_sentences)
    if "glat" in legs:
        result["glat_alignment"] = glat_timing(torch.randn(B, L, V, device=dev, generator=ggen).mul_(2).half(), targets, links, ol,
                                               cpu=(targets_cpu, links_cpu, m, n) if cpu else None)
    if "long" in legs:
        result["long_sentences"] = long_sentence_timing(dev)
    if "links" in legs:
        result["link_scorer"] = link_scorer_timing(dev)
    if "frontend" in legs:
        result["decode_front_end"] = decode_front_end_timing(dev)
    if "maxleft3" in legs:
        result["max_left_3"] = max_left3_timing(dev)
    if not args.no_cpu_baseline:
        batch_cpu = {"output_length": m, "target_length": n, "links": links_cpu, "targets": targets_cpu}
        result["cpu_baseline"] = cpu_baseline(batch_cpu, sample_logits, args.cpu_sentences)
        result["cpu_baseline"]["cpu_model"] = cpu_model_string()
        result["cpu_baseline"]["host_cpus"] = os.cpu_count()
        result["speedup_vs_cpu"] = result["value"] / result["cpu_baseline"]["value"]
        if "viterbi" in result and "cpu_b1" in result["viterbi"]:  # the second half of the metric, beside its CPU figures
            vit = result["viterbi"]
            result["cpu_baseline"]["viterbi"] = {
                "b1_ms_per_sentence": vit["cpu_b1"]["ms_per_sentence_mean"], "b1_decode_only_ms_per_sentence": vit["cpu_b1"]["decode_ms_mean"],
                "b1_cores": vit["cpu_b1"]["cores"], "b64_sentences_per_s": vit["cpu_b64"]["sentences_per_s_with_front_end"],
                "b64_decode_only_sentences_per_s": vit["cpu_b64"]["decode_only_sentences_per_s"], "b64_cores": vit["cpu_b64"]["cores"],
                "kind": "port", "sample": "all 1000 sentences of the inference configuration (the front-end on a strided sample of 16)",
                "gpu_b1_ms_per_sentence_mean": vit["b1"]["ms_per_sentence_mean"], "gpu_b64_sentences_per_s": vit["b64_sentences_per_s"]}
        if "glat_alignment" in result and "cpu" in result["glat_alignment"]:
            result["cpu_baseline"]["glat_alignment_ms_per_call"] = result["glat_alignment"]["cpu"]["ms_per_call"]
    print(json.dumps(result))


if __name__ == "__main__":
    main()

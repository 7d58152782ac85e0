"""Benchmark of one Bamboo pipeline stage on one MI355X.

A step is one ``train_batch`` of the stage (M micro-batches of own forward+backward through
the 1F1B instruction stream, the redundant forwards of the shadow layers, one fused Adam
step) over synthetic inputs that are resident in HBM before the timed region starts.

Prints ONE JSON line: ``value`` = samples/s with redundant computation ON (the configuration
the metric is quoted on), plus the RC-off rate and the RC overhead, a ``roofline`` object for
the dominant kernel (measured with HIP events around its launches inside the timed region)
and a ``cpu_baseline`` object (the CPU oracle timed on a bounded sample of the same workload).
"""
import argparse
import gc
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

CONFIGS = {
    # name: hidden, heads, ffn, layers per stage, seq, micro-batch, micro-batches, dtype, variant
    "c1": dict(hidden=768, heads=12, ffn=3072, layers=2, seq=512, mb=4, M=8, dtype="fp32",
               variant=dict(activation="gelu_tanh", ln="standard", mask="causal"), grad_mode="mse",
               label="GPT-2-small stage 2+2 layers h768 s512 mb4 M8 fp32"),
    "c2": dict(hidden=1024, heads=16, ffn=4096, layers=6, seq=1024, mb=8, M=16, dtype="bf16",
               variant=dict(activation="gelu_tanh", ln="standard", mask="causal"), grad_mode="queue",
               label="GPT-2-medium stage 6+6 layers h1024 s1024 mb8 M16 bf16"),
    "c3": dict(hidden=1024, heads=16, ffn=4096, layers=4, seq=512, mb=16, M=12, dtype="bf16",
               variant=dict(activation="gelu_tanh", ln="standard", mask="key_padding"), grad_mode="queue",
               key_len_range=(128, 512), label="BERT-large stage 4+4 layers h1024 s512 mb16 M12 bf16"),
    "c4": dict(kind="resnet", hidden=1024, mid=256, side=14, layers=12, seq=196, mb=32, M=8, dtype="bf16",
               grad_mode="queue", label="ResNet-152 conv4_x stage 12+12 bottleneck blocks 1024-256-256-1024 @14x14 mb32 M8 bf16 NHWC"),
    "c5": dict(hidden=1600, heads=25, ffn=6400, layers=8, seq=1024, mb=4, M=16, dtype="bf16",
               variant=dict(activation="gelu_tanh", ln="standard", mask="causal"), grad_mode="queue",
               label="GPT-2-1.5B stage 8+8 layers h1600 s1024 mb4 M16 bf16"),
}
STAGES, STAGE_ID = 4, 1
PEAK_BF16_TFLOPS, PEAK_F32_TFLOPS = 2500.0, 157.3

TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "gemm_bf16_dma_c2_gpt2_medium_stage_hbm_traffic.md")


def measured_traffic_bytes(config, kernel):
    """HBM bytes per launch of a GEMM variant as the two ``rocprofv3 --pmc`` runs summarised under profiles/ counted
    them (FETCH_SIZE and WRITE_SIZE, each scaled by what the same counter reads for a copy of known size).  Counters
    cannot be read from inside this process, so the figure is looked up in that summary's table ``| config | variant |
    bytes per launch |``; None for anything that was not profiled, or where the summary is not at hand."""
    try:
        for line in open(TRAFFIC_SUMMARY):
            cells = [c.strip().strip("`") for c in line.strip().strip("|").split("|")]
            if len(cells) == 3 and cells[0] == config and cells[1] == kernel and cells[2].isdigit():
                return int(cells[2])
    except OSError:
        pass
    return None


def build_engine(cfg, rc, rc_stream, seed=1138, use_graphs=False, paced=None, rc_issue="reference", eager=True,
                 stage_id=STAGE_ID):
    """``paced=(t_fwd, t_bwd)``: the neighbours are a closed-loop model of the other stages of a 1F1B pipeline whose
    forward / backward passes take that long, so the stage waits for its inputs as in a real pipeline.
    ``stage_id``: which stage of the ``STAGES`` is the real one (all stages have the same layers)."""
    import itertools

    import torch

    import bamboo_amd
    from bamboo_amd import BottleNeck, LayerSpec, MSELoss, PipelineModule, SeededActivationQueue, TransformerLayer
    from bamboo_amd.p2p import PacedActivationQueue
    dtype = torch.bfloat16 if cfg["dtype"] == "bf16" else torch.float32
    if cfg.get("kind") == "resnet":
        specs = [LayerSpec(BottleNeck, cfg["hidden"], cfg["mid"], height=cfg["side"], width=cfg["side"])
                 for _ in range(cfg["layers"] * STAGES)]
    else:
        specs = [LayerSpec(TransformerLayer, cfg["hidden"], cfg["heads"], cfg["ffn"], dropout=cfg.get("dropout", 0.0),
                           **cfg["variant"])
                 for _ in range(cfg["layers"] * STAGES)]
    # a stage that shadows the last one must be able to run it after a failover: the last stage carries the loss
    loss_fn = MSELoss() if stage_id + 1 == STAGES - 1 else None
    model = PipelineModule(specs, num_stages=STAGES, partition_method="uniform", stage_id=stage_id, dtype=dtype,
                           device="cuda:0", loss_fn=loss_fn)
    qargs = dict(stage_ids=[stage_id, stage_id + 1], seed=seed, grad_mode=cfg["grad_mode"], device="cuda:0",
                 key_len_range=cfg.get("key_len_range"))
    if paced is not None:
        q = PacedActivationQueue((cfg["mb"], cfg["seq"], cfg["hidden"]), dtype, cfg["M"], stages=STAGES, stage_id=stage_id,
                                 t_fwd=paced[0], t_bwd=paced[1], **qargs)
    else:
        q = SeededActivationQueue((cfg["mb"], cfg["seq"], cfg["hidden"]), dtype, cfg["M"], **qargs)
    ds = {"train_micro_batch_size_per_gpu": cfg["mb"], "gradient_accumulation_steps": cfg["M"],
          "optimizer": {"type": "Adam", "params": {"lr": 1e-3, "betas": [0.9, 0.999], "eps": 1e-8}},
          "bf16": {"enabled": cfg["dtype"] == "bf16"}}
    engine, _, _, _ = bamboo_amd.initialize(model=model, config=ds, redundancy_level=1 if rc else 0,
                                            eager_recovery=rc and eager, activation_queue=q, rc_stream=rc_stream,
                                            install_signal_handler=False, use_graphs=use_graphs, rc_issue=rc_issue)
    if stage_id == 0 or stage_id + 1 == STAGES - 1:
        # the first stage loads its input itself (LoadMicroBatch), and a stage that shadows the last one loads that
        # stage's labels: both come from the resident seeded tensors, micro-batch k of every batch the same
        engine.set_dataiterator(itertools.cycle([(a, a) for a in q.activations]))
    return engine, q


def measure_pass_times(engine, q):
    """Median GPU time of one forward and one backward pass of the stage's own layers (seconds), from events
    recorded behind every pass of one batch on an otherwise idle GPU: consecutive passes run back to back on one
    stream, so a pass lasts from the previous pass's end to its own."""
    import torch
    marks = []

    def note_done(kind, k, stage_id, stream):
        ev = torch.cuda.Event(enable_timing=True)
        ev.record(stream)
        marks.append((kind, ev))
    q.note_done = note_done
    torch.cuda.synchronize()
    base = torch.cuda.Event(enable_timing=True)
    base.record(torch.cuda.current_stream())
    engine.train_batch()
    torch.cuda.synchronize()
    del q.note_done
    durs = {"F": [], "B": []}
    prev = base
    for i, (kind, ev) in enumerate(marks):
        if i > 0:                        # the first pass also carries the start of the batch
            durs[kind].append(prev.elapsed_time(ev) * 1e-3)
        prev = ev
    med = lambda v: sorted(v)[len(v) // 2]
    return med(durs["F"]), med(durs["B"])


def paced_timeline(q, t_start):
    """Markdown rows of the stage's last batch inside the pipeline model: every own pass (when its input arrived,
    when it ran) and every piece of redundant forward work (when it ran, and beside which own pass, if any)."""
    c = q.clock
    sid = q.stage_id
    ms = lambda t: f"{(t - t_start) * 1e3:8.2f}"
    own, prev = [], c.t0
    for kind, k in c.order[sid]:
        arrive = c.activation_at(k) if kind == "F" else c.grad_at(k)
        end = c.end_of(sid, kind, k)
        own.append((f"{kind}{k}", arrive, max(arrive, prev), end))
        prev = end
    # pieces of one micro-batch's redundant forward that ran back to back are one row
    marks = [(k, layer, what, when()) for k, layer, what, when in q.rc_marks]
    pieces = []
    for (k, lo, _, t0), (_, hi, _, t1) in zip(marks[0::2], marks[1::2]):
        if pieces and pieces[-1][0] == k and pieces[-1][2] == lo and t0 - pieces[-1][4] < 50e-6:
            pieces[-1][2], pieces[-1][4] = hi, t1
        else:
            pieces.append([k, lo, hi, t0, t1])
    lines = ["| own pass | input arrived (ms) | started | ended | idle before it (ms) |", "|---|---:|---:|---:|---:|"]
    idle_total, last_end = 0.0, c.t0
    for name, arrive, start, end in own:
        idle_total += start - last_end
        lines.append(f"| {name} | {ms(arrive)} | {ms(start)} | {ms(end)} | {(start - last_end) * 1e3:6.2f} |")
        last_end = end
    lines += ["", f"Own stream idle inside the batch: {idle_total * 1e3:.2f} ms; pipeline end of the batch at {ms(c.pipeline_end())} ms.", "",
              "| redundant forward of micro-batch | layers | started (ms) | ended | overlapped with own passes (ms) | beside |", "|---|---|---:|---:|---:|---|"]
    in_idle = 0
    for k, lo, hi, t0, t1 in pieces:
        shared = [(name, max(0.0, min(t1, e) - max(t0, s))) for name, _, s, e in own]
        shared = [(n, d) for n, d in shared if d > 20e-6]
        ov = sum(d for _, d in shared)
        in_idle += ov < 0.1 * (t1 - t0)
        lines.append(f"| {k} | {lo}-{hi - 1} | {ms(t0)} | {ms(t1)} | {ov * 1e3:6.2f} of {(t1 - t0) * 1e3:5.2f} | {', '.join(n for n, _ in shared) or 'idle GPU'} |")
    lines += ["", f"{in_idle} of {len(pieces)} pieces ran with less than a tenth of their time beside an own pass."]
    return "\n".join(lines)


def own_pass_means(q):
    """Mean GPU duration (seconds) of the real stage's forward and backward passes in the batch the queue's clock
    holds: a pass runs from the later of its input's arrival and the previous pass's end to its own end, so time
    it shared with redundant work on the other stream is in it."""
    c, sid = q.clock, q.stage_id
    durs, prev = {"F": [], "B": []}, c.t0
    for kind, k in c.order[sid]:
        arrive = c.activation_at(k) if kind == "F" else c.grad_at(k)
        end = c.end_of(sid, kind, k)
        durs[kind].append(end - max(arrive, prev))
        prev = end
    return sum(durs["F"]) / len(durs["F"]), sum(durs["B"]) / len(durs["B"])


def paced_leg(cfg, rc, rc_issue, t_fwd, t_bwd, steps, warmup, timeline=None, stage_id=STAGE_ID):
    """Batch time (seconds, mean of ``steps`` batches) of the stage inside the closed-loop pipeline model, graphs on
    (one launch per pass: the host never holds the GPU back after a receive has returned)."""
    import torch
    work = torch.cuda.Stream()
    work.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(work):
        engine, q = build_engine(cfg, rc=rc, rc_stream=rc, use_graphs=True, paced=(t_fwd, t_bwd), rc_issue=rc_issue,
                                 stage_id=stage_id)
        for _ in range(max(warmup, 3)):      # eager batch, capturing batch, first replay
            engine.train_batch()
        q.reset()
        waits, per_batch = [], []
        for i in range(steps):
            if timeline is not None and i == steps - 1:
                q.rc_marks = []              # the last batch's redundant work, piece by piece
                t_start = q._last_end if i > 0 else 0.0
            engine.train_batch()
            waits.append(q.waited)
            per_batch.append(q.batch_seconds)
        total = q.finish()
        own_f, own_b = own_pass_means(q)
        if timeline is not None:
            with open(timeline, "w") as f:
                f.write(paced_timeline(q, t_start) + "\n")
    del engine, q
    gc.collect()
    torch.cuda.empty_cache()
    mean = lambda v: sum(v) / len(v)
    return {"batch_s": total / steps, "host_wait_s": mean(waits), "first_batch_s": per_batch[0],
            "later_batches_s": mean(per_batch[1:] or per_batch), "own_fwd_s": own_f, "own_bwd_s": own_b}


def paced_failure(cfg, rc_issue, t_fwd, t_bwd, at, stage_id):
    """The successor is lost at micro-batch ``at`` of a batch inside the pipeline model, redundant forwards issued
    as ``rc_issue`` says: how many shadow stashes the promoted stage finds missing (redundant forwards still held
    back, or issued in part) and has to compute first, and the pause (failure detected with the GPU drained ->
    the lost stage's work up to that point replayed)."""
    import torch
    engine, q = build_engine(cfg, rc=True, rc_stream=True, paced=(t_fwd, t_bwd), rc_issue=rc_issue, stage_id=stage_id)
    for _ in range(2):
        engine.train_batch()
    q.preempt_successor(at, stage_id)
    engine.train_batch()
    torch.cuda.synchronize()
    fo = engine.last_failover
    out = {"shadow_stashes_missing": fo["rc_missing"], "pause_ms": round(fo["pause_s"] * 1e3, 3),
           "detected_at_step": fo["step"]}
    del engine, q
    gc.collect()
    torch.cuda.empty_cache()
    return out


def paced_per_stage(cfg, t_fwd, t_bwd, steps, warmup, fail_at, known=None):
    """RC overhead inside the pipeline model with stage 0, 1, 2, ... of ``STAGES`` as the real one (the last stage
    shadows nobody in this build: redundancy ids are not wrapped round to stage 0's layers on another device).
    Every Bamboo stage runs redundant forwards, so for the RC-on legs the modelled neighbours get the pass times
    the real stage's own passes measure WITH its redundant work beside them (second leg, fed from the first);
    the RC-off leg uses the plain pass times for everybody.  The pipeline's figure is the worst stage's."""
    stages = {}
    for sid in range(STAGES - 1):
        off = (known or {}).get((sid, "off")) or paced_leg(cfg, False, "reference", t_fwd, t_bwd, steps, warmup, stage_id=sid)
        on1 = (known or {}).get((sid, "bubble")) or paced_leg(cfg, True, "bubble", t_fwd, t_bwd, steps, warmup, stage_id=sid)
        on2 = paced_leg(cfg, True, "bubble", on1["own_fwd_s"], on1["own_bwd_s"], steps, warmup, stage_id=sid)
        pct = lambda leg: round(100.0 * (leg["batch_s"] - off["batch_s"]) / off["batch_s"], 2)
        stages[str(sid)] = {
            "rc_off_batch_ms": round(off["batch_s"] * 1e3, 3),
            "rc_on_batch_ms_neighbours_plain": round(on1["batch_s"] * 1e3, 3),
            "rc_on_batch_ms_neighbours_with_rc": round(on2["batch_s"] * 1e3, 3),
            "own_pass_ms_with_rc": [round(on1["own_fwd_s"] * 1e3, 3), round(on1["own_bwd_s"] * 1e3, 3)],
            "rc_overhead_paced_pct_neighbours_plain": pct(on1),
            "rc_overhead_paced_pct": pct(on2),
            "failure_at_micro_batch": fail_at,
            "failure_bubble": paced_failure(cfg, "bubble", t_fwd, t_bwd, fail_at, sid),
            "failure_reference": paced_failure(cfg, "reference", t_fwd, t_bwd, fail_at, sid)}
    worst = max(stages, key=lambda k: stages[k]["rc_overhead_paced_pct"])
    return {"rc_issue": "bubble", "stages": stages, "pipeline_rc_overhead_paced_pct": stages[worst]["rc_overhead_paced_pct"],
            "worst_stage": int(worst),
            "note": "neighbours' passes in the RC-on figure take the real stage's mean pass times measured with its "
                    "redundant forwards beside them; pipeline figure = worst stage"}


def time_steps(engine, steps, warmup):
    import torch
    for _ in range(warmup):
        engine.train_batch()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        engine.train_batch()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


class GemmProbe:
    """Brackets every dense GEMM launch with HIP events on the launch stream."""

    def __init__(self):
        self.records = []

    def __call__(self, desc, launch, stream=None):
        import torch

        from bamboo_amd import hip
        if isinstance(desc, (list, tuple)):
            name = "grouped_" + hip.gemm_variant(desc[0]).rsplit("_", 1)[0]
            flops = sum(2.0 * d.M * d.N * d.K for d in desc)
            shape = "+".join(f"{d.M}x{d.N}x{d.K}" for d in desc)
        elif hasattr(desc, "variant_name"):      # implicit-GEMM convolution
            name, flops, shape = desc.variant_name, 2.0 * desc.M * desc.N * desc.K, f"{desc.M}x{desc.N}x{desc.K}"
        else:
            name, flops = hip.gemm_variant(desc), 2.0 * desc.M * desc.N * desc.K
            # an epilogue that evaluates the activation is a different code path with work of its own
            # (two transcendental-heavy outputs for act_dact): its launches are listed apart
            name += {hip.EPI_ACT: "+act", hip.EPI_DACT: "+dact", hip.EPI_ACT_DACT: "+act_dact"}.get(desc.epilogue, "")
            shape = f"{desc.M}x{desc.N}x{desc.K}"
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        stream = stream if stream is not None else torch.cuda.current_stream()
        e0.record(stream)        # on the stream the kernel is launched on
        launch()
        e1.record(stream)
        self.records.append((name, flops, e0, e1, shape))

    @staticmethod
    def bracket_overhead(n=200):
        """Seconds that an empty event bracket reads on an idle stream: what each bracket adds to
        the kernel it encloses (marker processing + dispatch), subtracted per launch in summary()."""
        import torch
        torch.cuda.synchronize()
        pairs = []
        for _ in range(n):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            e1.record()
            pairs.append((e0, e1))
        torch.cuda.synchronize()
        ts = sorted(a.elapsed_time(b) for a, b in pairs)
        return ts[len(ts) // 2] * 1e-3

    def by_shape(self):
        """{(variant, shape): [launches, flops, seconds]} for the --gemm-shapes table."""
        agg = {}
        for name, flops, e0, e1, shape in self.records:
            a = agg.setdefault((name, shape), [0, 0.0, 0.0])
            a[0] += 1
            a[1] += flops
            a[2] += e0.elapsed_time(e1) * 1e-3
        return agg

    def summary(self, overhead_s=0.0):
        """{variant: [launches, flops, seconds]}; ``overhead_s`` (an empty bracket's reading) is
        taken off every launch so that the durations are the kernels' own, as a kernel trace shows them."""
        agg = {}
        for name, flops, e0, e1, _ in self.records:
            a = agg.setdefault(name, [0, 0.0, 0.0])
            a[0] += 1
            a[1] += flops
            a[2] += max(e0.elapsed_time(e1) * 1e-3 - overhead_s, 1e-9)
        return agg


def cpu_baseline(cfg, threads):
    """Oracle stage on the host: one micro-batch of own forward+backward and one redundant
    forward at the benchmark's shapes (fp32), extrapolated to the batch."""
    import torch

    from oracle import layers as ol
    from oracle.stage import OracleStage
    torch.set_num_threads(threads)
    if cfg.get("kind") == "resnet":
        ocfg = ol.BottleneckCfg(in_channels=cfg["hidden"], mid_channels=cfg["mid"])
        cfg = dict(cfg, variant={"mask": "none"})
    else:
        ocfg = ol.TransformerCfg(hidden=cfg["hidden"], heads=cfg["heads"], ffn=cfg["ffn"], **cfg["variant"])
    parts = [i * cfg["layers"] for i in range(STAGES + 1)]
    st = OracleStage(ocfg, parts, STAGE_ID, cfg["M"], dtype=torch.float32, redundancy_level=1, eager=True)
    g = torch.Generator().manual_seed(1)
    x = torch.randn(cfg["mb"], cfg["seq"], cfg["hidden"], generator=g)
    dy = torch.randn(cfg["mb"], cfg["seq"], cfg["hidden"], generator=g)
    kl = None
    if cfg["variant"]["mask"] == "key_padding":
        kl = torch.randint(cfg["key_len_range"][0], cfg["key_len_range"][1] + 1, (cfg["mb"],), generator=g)
    reps = 2  # two micro-batches: about 10-15 s on 16 host cores at the c2 shapes
    t_own = t_rc = 0.0
    for _ in range(reps):
        t0 = time.perf_counter()
        xin = x.clone().requires_grad_(True)
        out = st.forward(xin, STAGE_ID, kl)
        torch.autograd.backward(out, dy)
        t_own += (time.perf_counter() - t0) / reps
        t0 = time.perf_counter()
        with torch.enable_grad():
            st.forward(out.detach().requires_grad_(True), STAGE_ID + 1, kl)
        t_rc += (time.perf_counter() - t0) / reps
    M = cfg["M"]
    samples = cfg["mb"] * M
    off, on = M * t_own, M * (t_own + t_rc)
    return {"value": samples / on, "unit": "samples/s", "cores": threads, "kind": "port",
            "rc_off_value": samples / off, "rc_overhead_pct": 100.0 * (on - off) / off,
            "sample": f"{reps} micro-batches, each own fwd+bwd ({t_own:.2f}s) + redundant fwd ({t_rc:.2f}s), fp32, "
                      f"mean extrapolated x{M} micro-batches; optimizer step not included"}


def failover_legs(cfg, engine, q, at, steps, warmup):
    """The successor is preempted at micro-batch ``at`` (reference path: the NextStageException branch of
    train_batch, engine.py:1190-1264).  ``engine`` has run warm-up and timed batches with redundant forwards (eager
    recovery); afterwards the same failure in lazy recovery (host mirrors of the shadow parameters, nothing computed
    ahead: promotion materialises the layers and the replay recomputes the successor's forwards)."""
    import torch
    samples = cfg["mb"] * cfg["M"]
    q.preempt_successor(at, STAGE_ID)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    engine.train_batch()
    torch.cuda.synchronize()
    t_fail_batch = time.perf_counter() - t0
    q.revive()
    t_post = time_steps(engine, steps, 1)       # merged own+promoted stream from step 0
    fo = engine.last_failover
    failover = {"preempted_at_micro_batch": at, "detected_at_step": fo["step"],
                "promote_ms": round(fo["promote_s"] * 1e3, 3), "pause_ms": round(fo["pause_s"] * 1e3, 3),
                "shadow_stashes_missing": fo["rc_missing"],
                "failover_batch_ms": round(t_fail_batch * 1e3, 3),
                "post_failover_samples_per_s": round(samples / t_post, 3),
                "post_failover_ms_per_step": round(t_post * 1e3, 3),
                "note": "pause = failure detected (GPU drained) -> successor's lost work replayed from the RC stash; "
                        "post-failover = own + promoted layers as two local stages"}
    del engine, q
    gc.collect()
    torch.cuda.empty_cache()
    engine, q = build_engine(cfg, rc=True, rc_stream=False, eager=False)
    t_lazy = time_steps(engine, steps, warmup)
    q.preempt_successor(at, STAGE_ID)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    engine.train_batch()
    torch.cuda.synchronize()
    t_fail_lazy = time.perf_counter() - t0
    q.revive()
    fo = engine.last_failover
    failover["lazy"] = {"samples_per_s_before": round(samples / t_lazy, 3), "promote_ms": round(fo["promote_s"] * 1e3, 3),
                        "pause_ms": round(fo["pause_s"] * 1e3, 3), "failover_batch_ms": round(t_fail_lazy * 1e3, 3),
                        "note": "redundancy_level=1 without eager recovery: no RC overhead before the failure, the "
                                "pause pays for building the layers from host mirrors and for the lost forwards"}
    del engine, q
    gc.collect()
    torch.cuda.empty_cache()
    return failover


def dominant_gemm(probe, dtype):
    """(name, launches, flops, seconds, all variants) of the GEMM variant with the largest total time."""
    overhead_s = probe.bracket_overhead()
    agg = probe.summary(overhead_s)
    name, (count, flops, secs) = max(agg.items(), key=lambda kv: kv[1][2])
    return name, count, flops, secs, agg, overhead_s


def quick_config(name, steps, warmup, failover_at=None, dropout=None):
    """A bounded run of another configuration with the same code: RC off, RC on (second stream), the dominant GEMM
    variant's rate from event brackets on a single-stream RC-on leg, optionally the failover figures."""
    import torch
    cfg = CONFIGS[name]
    if dropout:
        cfg = dict(cfg, dropout=dropout)
    samples = cfg["mb"] * cfg["M"]
    peak = PEAK_BF16_TFLOPS if cfg["dtype"] == "bf16" else PEAK_F32_TFLOPS

    def drop(engine, q):
        del engine, q
        gc.collect()
        torch.cuda.empty_cache()
    engine, q = build_engine(cfg, rc=False, rc_stream=False)
    t_off = time_steps(engine, steps, warmup)
    drop(engine, q)
    out = {"workload": cfg["label"], "dtype": cfg["dtype"], "steps": steps, "warmup": warmup, "samples_per_step": samples,
           "dropout": cfg.get("dropout", 0.0)}
    if dropout is None:
        engine, q = build_engine(cfg, rc=True, rc_stream=False)
        for _ in range(warmup):
            engine.train_batch()
        probe = GemmProbe()
        engine.set_gemm_hook(probe)
        for _ in range(steps):
            engine.train_batch()
        torch.cuda.synchronize()
        engine.set_gemm_hook(None)
        drop(engine, q)
        kname, count, flops, secs, _, _ = dominant_gemm(probe, cfg["dtype"])
        out["dominant_kernel"] = {"kernel": f"gemm_{kname}", "launches": count, "avg_launch_us": round(secs / count * 1e6, 2),
                                  "achieved_tflops": round(flops / secs / 1e12, 2), "peak_tflops": peak,
                                  "frac": round(flops / secs / 1e12 / peak, 4)}
    engine, q = build_engine(cfg, rc=True, rc_stream=True)
    t_on = time_steps(engine, steps, warmup)
    out.update({"rc_on_samples_per_s": round(samples / t_on, 3), "rc_off_samples_per_s": round(samples / t_off, 3),
                "rc_overhead_pct": round(100.0 * (t_on - t_off) / t_off, 2), "ms_per_step_rc_on": round(t_on * 1e3, 3)})
    if failover_at is not None:
        out["failover"] = failover_legs(cfg, engine, q, failover_at, steps, warmup)
        engine = q = None
    else:
        drop(engine, q)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--config", default="c2", choices=sorted(CONFIGS))
    ap.add_argument("--rc-stream", type=int, default=1, help="issue redundant forwards on a second HIP stream")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-probe", action="store_true", help="do not bracket GEMM launches with events")
    ap.add_argument("--gemm-shapes", action="store_true", help="print a per-shape GEMM table on stderr")
    ap.add_argument("--skip-rc-off", action="store_true")
    ap.add_argument("--graphs", type=int, default=0,
                    help="replay each micro-batch's forward/backward launch sequence as a HIP graph in the RC-off leg and "
                         "in the leg `value` is quoted on (captured during warm-up; the probed leg always launches eagerly); "
                         "off by default: at these shapes the GPU is never waiting for the host, so it measures the same")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="first run three 256 MiB fp32 copies (cast_kernel<float,float>): the known-size kernel that "
                         "FETCH_SIZE / WRITE_SIZE counters of a --pmc run are scaled by")
    ap.add_argument("--dropout", type=float, default=0.0,
                    help="dropout probability of the transformer layers (the reference scripts run 0.1; the benchmark "
                         "line is quoted at 0, the configuration names none)")
    ap.add_argument("--script-layers", action="store_true",
                    help="the layer variant of the reference's transformer script (ReLU, annotated LayerNorm, no mask) "
                         "at the configuration's sizes, instead of its GPT-2 / BERT variant")
    ap.add_argument("--no-paced", action="store_true",
                    help="skip the legs that run the stage inside the closed-loop model of a 4-stage 1F1B pipeline")
    ap.add_argument("--paced-timeline", default=None, metavar="FILE",
                    help="write the last batch of the paced 'bubble' leg as a table: own passes and pieces of redundant work")
    ap.add_argument("--failover-at", type=int, default=None,
                    help="also measure a failover: the successor is preempted at this micro-batch (config c5: 7)")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="only the configuration --config names: leave out the bounded runs of the other configurations "
                         "(3 batches each; GPT-2-1.5B with a failover at micro-batch 7), the per-stage legs of the "
                         "pipeline model and the dropout 0.1 rates that the default run appends")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures ONE pipeline stage on ONE GPU; --gpus N>1 is not part of this build", file=sys.stderr)
        sys.exit(2)

    import torch

    from bamboo_amd import hip
    cfg = CONFIGS[args.config]
    if args.script_layers:
        if "variant" not in cfg:
            print("bench.py: --script-layers goes with the transformer configurations", file=sys.stderr)
            sys.exit(2)
        cfg = dict(cfg, variant=dict(activation="relu", ln="annotated", mask="none"),
                   label=cfg["label"] + " (script layers: relu, annotated LayerNorm, no mask)")
        cfg.pop("key_len_range", None)
    if args.dropout > 0.0:
        # keys change every batch, so no HIP graphs, and the paced legs (which replay graphs) are left out
        if args.graphs or cfg.get("kind") == "resnet":
            print("bench.py: --dropout goes with the transformer configurations and without --graphs", file=sys.stderr)
            sys.exit(2)
        cfg = dict(cfg, dropout=args.dropout)
        args.no_paced = True
    samples = cfg["mb"] * cfg["M"]
    graphs = bool(args.graphs)
    if graphs:
        # graphs are captured from a created stream (the default stream cannot be captured), in the
        # second warm-up batch: the first one launches every kernel eagerly
        args.warmup = max(args.warmup, 2)
        work_stream = torch.cuda.Stream()
        work_stream.wait_stream(torch.cuda.current_stream())
        torch.cuda.set_stream(work_stream)
    if args.calibrate_copy:
        src = torch.ones(64 * 1024 * 1024, dtype=torch.float32, device="cuda:0")
        dst = torch.empty_like(src)
        for _ in range(3):
            hip.cast(src, dst)
        torch.cuda.synchronize()
        del src, dst

    # leg 1: RC off (plain 1F1B stream of the stage)
    t_off = None
    pass_times = None
    if not args.skip_rc_off:
        engine, q = build_engine(cfg, rc=False, rc_stream=False, use_graphs=graphs)
        t_off = time_steps(engine, args.steps, args.warmup)
        if not args.no_paced:
            pass_times = measure_pass_times(engine, q)
        del engine, q
        gc.collect()      # engines hold reference cycles (schedule generators, captured graphs)
        torch.cuda.empty_cache()

    # leg 2: RC on, everything on one stream; GEMM launches are bracketed with events here, where
    # no other stream shares the GPU, so the durations are the kernels' own
    engine, q = build_engine(cfg, rc=True, rc_stream=False)
    probe = None
    t_on_serial = time_steps(engine, args.steps, args.warmup)      # the leg's own rate, no event brackets
    if not args.no_probe:
        # the same steps again with every GEMM launch bracketed (costs ~10 % of the rate: not what is reported)
        probe = GemmProbe()
        engine.set_gemm_hook(probe)
        for _ in range(args.steps):
            engine.train_batch()
        torch.cuda.synchronize()
        engine.set_gemm_hook(None)
    t_on = t_on_serial

    # leg 3 (default): RC on with the redundant forwards on a second HIP stream; this is the
    # configuration `value` is quoted on
    if args.rc_stream:
        del engine, q
        gc.collect()      # engines hold reference cycles (schedule generators, captured graphs)
        torch.cuda.empty_cache()
        engine, q = build_engine(cfg, rc=True, rc_stream=True, use_graphs=graphs)
        t_on = time_steps(engine, args.steps, args.warmup)

    n_graphs = sum(1 for v in engine._graphs.values() if isinstance(v, tuple))
    fwd_flops_layer = engine.module.func_buckets[STAGE_ID][0].flops_fwd(cfg["mb"], cfg["seq"])
    failover = None
    if args.failover_at is not None:
        failover = failover_legs(cfg, engine, q, args.failover_at, args.steps, args.warmup)
    engine = q = None
    gc.collect()
    torch.cuda.empty_cache()

    fwd_flops = fwd_flops_layer * cfg["layers"]
    own_flops, rc_flops = 3 * fwd_flops * cfg["M"], fwd_flops * cfg["M"]

    roofline = None
    if probe is not None:
        name, count, flops, secs, agg, overhead_s = dominant_gemm(probe, cfg["dtype"])
        if args.gemm_shapes:
            for (vname, shape), (n, fl, sec) in sorted(probe.by_shape().items(), key=lambda kv: -kv[1][2]):
                print(f"{vname:34s} {shape:40s} n={n:5d} {sec / n * 1e6:8.1f} us {fl / sec / 1e12:7.1f} TF {sec * 1e3:8.2f} ms",
                      file=sys.stderr)
        peak = PEAK_BF16_TFLOPS if cfg["dtype"] == "bf16" else PEAK_F32_TFLOPS
        achieved = flops / secs / 1e12
        roofline = {"bound": "mfma", "achieved": round(achieved, 2), "peak": peak, "unit": "TFLOP/s",
                    "frac": round(achieved / peak, 4),
                    "traffic": measured_traffic_bytes(args.config, f"gemm_{name}"), "kernel": f"gemm_{name}",
                    "measured_in": "a repeat of the timed steps of the RC-on single-stream leg with HIP events around "
                                   "each GEMM launch on its stream, minus the reading of an empty event bracket",
                    "event_bracket_overhead_us": round(overhead_s * 1e6, 2),
                    "launches": count, "avg_launch_us": round(secs / count * 1e6, 2),
                    "avg_launch_gflop": round(flops / count / 1e9, 3),
                    "all_gemm_variants": {k: {"launches": v[0], "tflops": round(v[1] / v[2] / 1e12, 2),
                                              "time_s": round(v[2], 4)} for k, v in agg.items()}}

    out = {
        "metric": "stage samples/s RC on vs off, RC overhead %, MFMA util % (GPT-2-med stage)",
        "value": round(samples / t_on, 3), "unit": "samples/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(t_on * 1e3, 3), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": cfg["dtype"], "data": "synthetic",
        "config": {"workload": cfg["label"], "stage": f"{STAGE_ID} of {STAGES}", "redundancy_level": 1,
                   "eager_recovery": True, "rc_stream": bool(args.rc_stream), "hip_graphs": n_graphs if graphs else 0,
                   "samples_per_step": samples, "dropout": cfg.get("dropout", 0.0),
                   "attention": "n/a (convolutions as GEMMs over NHWC rows, 3x3 as implicit GEMMs)" if cfg.get("kind") == "resnet"
                   else ("unfused (fp32: scores and probabilities in HBM, as the reference); flops counted dense" if cfg["dtype"] == "fp32"
                         else "fused (no score matrix in HBM); flops counted dense, the causal kernel skips masked tiles")},
        "rc_on_samples_per_s": round(samples / t_on, 3),
        "rc_off_samples_per_s": None if t_off is None else round(samples / t_off, 3),
        "rc_overhead_pct": None if t_off is None else round(100.0 * (t_on - t_off) / t_off, 2),
        "rc_on_single_stream_samples_per_s": round(samples / t_on_serial, 3),
        "rc_overhead_single_stream_pct": None if t_off is None else round(100.0 * (t_on_serial - t_off) / t_off, 2),
        "stage_tflops_rc_on": round((own_flops + rc_flops) / t_on / 1e12, 2),
        "stage_tflops_rc_off": None if t_off is None else round(own_flops / t_off / 1e12, 2),
        "roofline": roofline,
    }
    if t_off is not None:
        # What the same work costs inside a real S-stage 1F1B pipeline, where each stage idles for
        # (S-1) forward+backward slots per batch and the redundant forwards fall into that idle time
        # (lock-step model; slot = t_off / M): only the part of the RC time that exceeds the bubbles delays
        # the batch.  Modelled from the measured times above, not measured itself.
        slot = t_off / cfg["M"]
        idle = (STAGES - 1) * slot
        model = lambda t_with_rc: round(100.0 * max(0.0, (t_with_rc - t_off) - idle) / (t_off + idle), 2)
        out["rc_overhead_bubble_model_pct"] = {"stages": STAGES, "single_stream": model(t_on_serial),
                                               "second_stream": model(t_on)}
    if pass_times is not None:
        # The stage inside a pipeline that has bubbles: the other three stages are a closed-loop model (their passes
        # take what this stage's own passes take, they react to what this stage really sends and when), receives
        # wait on the host until the model delivers.  RC off and RC on run under the same model; the redundant
        # forwards go to the second stream either where the reference places them or as soon as their input exists.
        t_fwd, t_bwd = pass_times
        off = paced_leg(cfg, False, "reference", t_fwd, t_bwd, args.steps, args.warmup)
        legs = {issue: paced_leg(cfg, True, issue, t_fwd, t_bwd, args.steps, args.warmup,
                                 timeline=args.paced_timeline if issue == "bubble" else None)
                for issue in ("reference", "asap", "bubble")}
        best = min(legs, key=lambda k: legs[k]["batch_s"])
        pct = lambda leg: round(100.0 * (leg["batch_s"] - off["batch_s"]) / off["batch_s"], 2)
        r3 = lambda d: {k: round(v * 1e3, 3) for k, v in d.items()}
        out["rc_overhead_paced_pct"] = pct(legs[best])
        out["paced"] = {
            "model": f"closed-loop {STAGES}-stage 1F1B, stage {STAGE_ID} real, neighbours' passes = this stage's measured "
                     "forward/backward, host-side waits, HIP graphs; batches back to back (a batch starts when the pipeline has finished the "
                     "previous one), batch_s = (start of the first batch -> max(pipeline end of the last, own GPU work drained)) / steps",
            "t_fwd_ms": round(t_fwd * 1e3, 3), "t_bwd_ms": round(t_bwd * 1e3, 3),
            "ideal_batch_ms": round((cfg["M"] + STAGES - 1) * (t_fwd + t_bwd) * 1e3, 3),
            "rc_off_ms": r3(off), "rc_on_reference_ms": r3(legs["reference"]), "rc_on_asap_ms": r3(legs["asap"]), "rc_on_bubble_ms": r3(legs["bubble"]),
            "rc_overhead_reference_pct": pct(legs["reference"]), "rc_overhead_asap_pct": pct(legs["asap"]),
            "rc_overhead_bubble_pct": pct(legs["bubble"]),
            "rc_issue_quoted": best,
            "rc_off_samples_per_s": round(samples / off["batch_s"], 3),
            "rc_on_samples_per_s": round(samples / legs[best]["batch_s"], 3)}
    if failover is not None:
        out["failover"] = failover
    extras = not args.no_other_configs and args.config == "c2" and args.dropout == 0.0 and not args.script_layers
    if extras and pass_times is not None:
        # every stage of the pipeline runs redundant forwards: the pipeline's overhead is the worst stage's
        known = {(STAGE_ID, "off"): off, (STAGE_ID, "bubble"): legs["bubble"]}
        out["paced_per_stage"] = paced_per_stage(cfg, t_fwd, t_bwd, args.steps, args.warmup, fail_at=7, known=known)
    if extras:
        # the configuration the reference's scripts train with (dropout 0.1 at all four sites of a layer)
        d = quick_config("c2", 3, 1, dropout=0.1)
        out["dropout_0p1"] = {k: d[k] for k in ("rc_on_samples_per_s", "rc_off_samples_per_s", "rc_overhead_pct", "steps")}
        other = {}
        for name in ("c1", "c3", "c4", "c5"):
            other[name] = quick_config(name, 3, 1, failover_at=7 if name == "c5" else None)
        out["other_configs"] = other
    if not args.no_cpu_baseline:
        # all host cores this process may run on (the affinity mask is what the box really grants; os.cpu_count()
        # reports the machine's)
        threads = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
        if os.environ.get("OMP_NUM_THREADS", "").isdigit():
            # a GPU box exports its CPU share of the host here; more threads than that would be time-sliced
            threads = min(threads, int(os.environ["OMP_NUM_THREADS"]))
        out["cpu_baseline"] = cpu_baseline(cfg, threads)
    print(json.dumps(out))


if __name__ == "__main__":
    main()

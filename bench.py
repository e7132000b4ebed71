#!/usr/bin/env python3
"""Headline benchmark: samples/s of one PipeDream stage's steady-state 1F1B step
(forward + backward + stashed SGD update) on one MI355X.

Workload (N=1): VGG16 conv1_1..pool2, batch 64 fp32, synthetic N(0,1) images, He-normal
weights, weight-stash depth 4 (3 warm-up forwards in flight), SGD momentum 0.9 lr 0.01
wd 5e-4; the stage is driven through StageRuntime / SGDWithWeightStashing and this script
plays its downstream neighbour (consumes the sent activation, queues a synthetic upstream
gradient ~ N(0,1)*1e-3).  All inputs are resident in HBM before the timed region.

Prints ONE JSON line (see the keys below).  `roofline` covers the dominant kernel, the
MFMA fp32 3x3 convolution by Winograd F(2x2, 3x3) (`winograd_fwd_kernel`, used for forward
and input gradient): algorithmic flop of its launches in the timed region (those of the
direct convolution, 2*9*C*K per output pixel) / their summed duration, both measured with
HIP events around every launch on the launch stream.  The kernel issues 16/36 of those
multiplications to the MFMA units: `roofline.achieved` / `roofline.frac` are the rate it actually
executes against the MFMA fp32 peak (never above 1), `roofline.direct_equivalent` is the rate a direct
convolution would need for the same launch time.  `roofline.traffic` is read from the tracked summary of
the rocprofv3 --pmc runs under profiles/ and is refused if that summary is about another kernel.
`cpu_baseline` times the CPU oracle (torch.nn on the host cores) on a bounded sample of
the same workload.

`--workload vgg16_pipeline | gnmt | gnmt_criterion | transformer` print the same kind of line for the
other configurations (full VGG16 as four co-resident stages; the LSTM stage; the GNMT classifier +
criterion; the 2BW transformer stage), each with its own CPU baseline sample.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

BATCH = 64
STASH_DEPTH = 4
SGD_KW = dict(lr=0.01, momentum=0.9, weight_decay=5e-4)
PEAK_FP32_MFMA_TFLOPS = 157.3
# HBM bytes per launch of the dominant kernel: written next to the summary of the rocprofv3 --pmc
# FETCH_SIZE / WRITE_SIZE runs it comes from
TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "winograd_fwd_vgg16_front_stage_bs64_pmc_traffic.json")


def measured_traffic(kernel):
    """HBM bytes per launch of ``kernel`` from the tracked counter summary, None if there is none; a summary
    that is about another kernel is an error, not a number to print."""
    if not os.path.isfile(TRAFFIC_SUMMARY):
        return None
    with open(TRAFFIC_SUMMARY) as f:
        rec = json.load(f)
    if rec["kernel"] != kernel:
        sys.exit("bench.py: %s holds the HBM traffic of %r, the timed kernel is %r; profile the current kernel "
                 "again (bench.py --pmc-probe under rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE) or remove the file"
                 % (TRAFFIC_SUMMARY, rec["kernel"], kernel))
    return float(rec["traffic_bytes_per_launch"])


def build_stage():
    import torch
    from pipedream_amd import handoff, runtime, sgd
    from pipedream_amd.layers import CrossEntropyLoss
    from pipedream_amd.stages import vgg16

    handoff.reset_fabrics()
    torch.manual_seed(0)

    class Rest(torch.nn.Module):     # placeholder for the stages that follow; never run
        def forward(self, x):
            raise RuntimeError("downstream stages are played by the benchmark")

    model = [(vgg16.FrontStage(), ["input0"], ["out0"]), (Rest(), ["out0"], ["out1"]),
             (CrossEntropyLoss(), ["out1"], ["loss"])]
    shapes = {"input0": (BATCH, 3, 224, 224), "target": (BATCH,), "out0": (BATCH, 128, 56, 56)}
    dtypes = {"input0": torch.float32, "target": torch.int64, "out0": torch.float32}
    r = runtime.StageRuntime(
        model=model, distributed_backend="gloo", fp16=False, loss_scale=1.0,
        training_tensor_shapes=shapes, eval_tensor_shapes=dict(shapes), training_tensor_dtypes=dtypes,
        inputs_module_destinations={"input": 0}, target_tensor_names={"target"},
        configuration_maps={"module_to_stage_map": [0, 1, 1], "stage_to_rank_map": {"0": [0], "1": [1]},
                            "stage_to_depth_map": {"0": STASH_DEPTH - 1, "1": 0}},
        master_addr="127.0.0.1", rank=0, local_rank=0, num_ranks_in_server=2, verbose_freq=0,
        model_type=runtime.IMAGE_CLASSIFICATION)
    opt = sgd.SGDWithWeightStashing(r.modules(), r.master_parameters, r.model_parameters, 1.0,
                                    num_versions=r.num_warmup_minibatches + 1, **SGD_KW)
    return r, opt


class Downstream(object):
    """The next stage as seen from the hand-off queues."""

    def __init__(self, r, grads):
        self.fabric = r.comm_handler.fabric
        self.grads = grads
        self.i = 0

    def after_forward(self):
        self.fabric.take("out0", 1, False)
        self.fabric.take("target", 1, False)
        self.fabric.put("out0", 0, True, self.grads[self.i % len(self.grads)])
        self.i += 1


def gpu_run(steps, warmup):
    import torch
    from pipedream_amd import ops

    r, opt = build_stage()
    g = torch.Generator().manual_seed(0)
    n_data = 4
    images = [torch.randn(BATCH, 3, 224, 224, generator=g).cuda().contiguous(memory_format=torch.channels_last)
              for _ in range(n_data)]
    targets = [torch.randint(0, 1000, (BATCH,), generator=g).cuda() for _ in range(n_data)]
    grads = [(torch.randn(BATCH, 128, 56, 56, generator=g) * 1e-3).cuda().contiguous(
        memory_format=torch.channels_last) for _ in range(n_data)]

    def loader():
        i = 0
        while True:
            yield images[i % n_data], targets[i % n_data]
            i += 1

    total = warmup + steps + r.num_warmup_minibatches
    r.train(total)
    r.set_loader(loader())
    down = Downstream(r, grads)

    def forward():
        r.run_forward()
        down.after_forward()

    def step():
        forward()
        opt.zero_grad()
        opt.load_old_params()
        r.run_backward()
        opt.load_new_params()
        opt.step()

    for _ in range(r.num_warmup_minibatches):     # fill the pipeline: 3 forwards in flight
        forward()
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    ops.kernel_timer = {}
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    timer, ops.kernel_timer = ops.kernel_timer, None

    stats = {}
    for name, recs in timer.items():
        ms = sum(s.elapsed_time(e) for s, e, _ in recs)
        stats[name] = {"launches": len(recs), "avg_us": 1e3 * ms / len(recs),
                       "work_per_launch": sum(w for _, _, w in recs) / len(recs),
                       "rate": sum(w for _, _, w in recs) / (ms * 1e-3)}
    done = warmup + steps
    assert opt.queue.versions() == [done - (STASH_DEPTH - 1) + i for i in range(STASH_DEPTH)], opt.queue.versions()
    return elapsed, stats, opt


def pmc_probe():
    """Workload for `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE` runs: a plain copy of
    known size (calibrates the counters: pd_copy_kernel moves 1 GiB in and 1 GiB out per
    launch) followed by steady-state steps of the benchmark stage, so the per-dispatch counter values of
    the convolution kernels cover exactly the launch mix of the timed region, and by the optimizer kernel
    on the VGG16-sized parameter set.  The same workload serves the MFMA-utilisation counters."""
    import ctypes
    import torch
    from pipedream_amd import _cabi
    n = 1 << 30
    src = torch.empty(n, dtype=torch.uint8, device="cuda").fill_(1)
    dst = torch.empty(n, dtype=torch.uint8, device="cuda")
    for _ in range(3):
        _cabi.lib().pd_copy(ctypes.c_void_p(dst.data_ptr()), ctypes.c_void_p(src.data_ptr()), n, _cabi.stream_ptr())
    torch.cuda.synchronize()
    del src, dst
    gpu_run(steps=2, warmup=1)
    # and the fused stash + SGD kernel on the VGG16 parameter set of `optimizer_hbm`
    optimizer_bandwidth("SGD")
    print("pmc probe done")


def optimizer_bandwidth(kind="SGD"):
    """The fused stash + optimizer step as the product runs it: SGDWithWeightStashing (or the Adam wrapper)
    over the parameters of all four VGG16 stages (138 357 544 fp32 values in 32 tensors) with two weight
    versions, so every step reads the live ring slot and writes the other one.  20 (SGD) / 28 (Adam)
    algorithmic bytes per parameter; timed with HIP events on the launch stream over 20 steps."""
    import torch
    from pipedream_amd import adam, sgd
    from pipedream_amd.layers import CrossEntropyLoss
    from pipedream_amd.stages import vgg16
    torch.manual_seed(0)
    mods = [m.cuda() for m, _, _ in vgg16.model(CrossEntropyLoss())[:4]]
    params = [p for m in mods for p in m.parameters()]
    n = sum(p.numel() for p in params)
    if kind == "SGD":
        opt, bpp = sgd.SGDWithWeightStashing(mods, params, None, 1.0, 2, **SGD_KW), 20
    else:
        opt, bpp = adam.AdamWithWeightStashing(mods, params, None, 1.0, 2, lr=1e-3, betas=(0.9, 0.999)), 28
    for p in params:
        p.grad = torch.randn_like(p)
    for _ in range(3):
        opt.step()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    reps = 20
    torch.cuda.synchronize()
    e0.record()
    for _ in range(reps):
        opt.step()
    e1.record()
    torch.cuda.synchronize()
    sec = e0.elapsed_time(e1) * 1e-3 / reps
    assert opt.latest_version.version == reps + 3
    return {"kernel": "pd_optim_kernel<%s>" % kind, "params": n, "tensors": len(params), "bytes_per_param": bpp,
            "avg_us": sec * 1e6, "achieved_GBps": bpp * n / sec / 1e9, "peak_GBps": 8000.0,
            "frac": bpp * n / sec / 1e9 / 8000.0}


def cpu_baseline(timed_steps=6):
    """The CPU oracle (torch.nn modules, state_dict-copy weight stashing, torch.optim.SGD)
    on the same workload: 1 warm-up + `timed_steps` steady-state steps at batch 64."""
    import torch
    from oracle import models, stash_oracle
    torch.manual_seed(0)
    m = models.VggFrontStage()
    opt = stash_oracle.StashingOptimizerOracle("SGD", [m], m.parameters(), STASH_DEPTH, **SGD_KW)
    g = torch.Generator().manual_seed(0)
    x = torch.randn(BATCH, 3, 224, 224, generator=g)
    grad = torch.randn(BATCH, 128, 56, 56, generator=g) * 1e-3
    pending = [m(x) for _ in range(STASH_DEPTH - 1)]

    def step():
        pending.append(m(x))
        opt.zero_grad()
        opt.load_old_params()
        pending.pop(0).backward(grad)
        opt.load_new_params()
        opt.step()

    step()
    t0 = time.perf_counter()
    for _ in range(timed_steps):
        step()
    sec = (time.perf_counter() - t0) / timed_steps
    return {"value": BATCH / sec, "unit": "samples/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": "%d steady-state steps at batch 64 after 1 warm-up step (%.1f s/step)" % (timed_steps, sec)}


# ---- other configurations (not the default line): one stage each, same step definition ----------

def _run_steps(step, steps, warmup, before_instrumented=None):
    """Throughput over `steps` un-instrumented steps, then a short instrumented pass for the per-kernel
    figures (an event pair around each of the thousands of launches of these stages would slow the
    timed region itself).  `before_instrumented` is called between the two (a stage that runs passes of
    different minibatches side by side goes back to one stream there, so that a launch's duration is the
    kernel's own)."""
    import torch
    from pipedream_amd import ops
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    if before_instrumented is not None:
        before_instrumented()
        step()                      # one step to settle on the new stream arrangement, outside the event pairs
        torch.cuda.synchronize()
    ops.kernel_timer = {}
    for _ in range(min(steps, 4)):
        step()
    torch.cuda.synchronize()
    timer, ops.kernel_timer = ops.kernel_timer, None
    stats = {}
    for name, recs in timer.items():
        ms = sum(s.elapsed_time(e) for s, e, _ in recs)
        stats[name] = {"launches": len(recs), "avg_us": round(1e3 * ms / len(recs), 1),
                       "TFLOP/s": round(sum(w for _, _, w in recs) / (ms * 1e-3) / 1e12, 2)}
    return elapsed, stats


def gnmt_run(steps, warmup, overlap=True):
    """Embedding (32320 x 1024) + 4 LSTM layers (hidden 1024, residuals), T = 50, batch 128, fp32,
    AdamWithWeightStashing with stash depth 3 (2 forwards in flight)."""
    import contextlib
    import torch
    from pipedream_amd import adam, schedule
    from pipedream_amd.stages import gnmt
    torch.manual_seed(0)
    m = gnmt.Stage0(dropout=0.0).cuda()
    opt = adam.AdamWithWeightStashing([m], list(m.parameters()), None, 1.0, 3, lr=1e-3, betas=(0.9, 0.999))
    ids = torch.randint(0, 32320, (50, 128)).cuda()
    dy = (torch.randn(50, 128, 1024) * 1e-2).cuda()
    # minibatch j runs on stream j mod 3: the forward recurrence of minibatch k + 2 beside the backward
    # recurrence of minibatch k (schedule.MinibatchStreams; same results as one stream, bit for bit)
    rings = [schedule.MinibatchStreams(2) if overlap else None]
    if rings[0] is not None:
        rings[0].join()
    count = {"f": 0, "b": 0}
    pend = []

    def one_stream():
        if rings[0] is not None:
            rings[0].leave()
            rings[0] = None

    def forward():
        ring = rings[0]
        with (ring.forward(count["f"]) if ring is not None else contextlib.nullcontext()):
            pend.append(m(ids))
        count["f"] += 1

    def step():
        forward()
        ring = rings[0]
        with (ring.backward(count["b"]) if ring is not None else contextlib.nullcontext()):
            opt.zero_grad()
            opt.load_old_params()
            pend.pop(0).backward(dy)
            opt.load_new_params()
            opt.step()
        count["b"] += 1

    forward()
    forward()
    elapsed, stats = _run_steps(step, steps, warmup, one_stream)
    return elapsed, stats, 128, "f32", ("GNMT-style stage: embedding 32320x1024 + 4 LSTM layers hidden 1024 with residuals, "
                                         "seq 50, batch 128, fp32, Adam, stash depth 3"
                                         + (", forward of a new minibatch beside the backward of the oldest (one stream "
                                            "per minibatch in flight)" if overlap else ", one stream"))


def transformer_run(steps, warmup, overlap=True):
    """6 pre-LN transformer layers (hidden 1024, 16 heads, FFN 4096), micro-batch 8 x 512 tokens,
    bf16 compute, fp32 master weights + Adam every 4 micro-batches, 2 weight versions.  One step =
    one micro-batch forward + backward (+ the update on every 4th)."""
    import contextlib
    import torch
    from pipedream_amd import adam, schedule
    from pipedream_amd.stages import transformer
    torch.manual_seed(0)
    m = transformer.Stage0().cuda()
    opt = adam.AdamWithWeightStashing([m], list(m.parameters()), None, 1.0, 2, update_interval=4, bf16_image=True,
                                      lr=1e-3, betas=(0.9, 0.999))
    x = torch.randn(8, 512, 1024).cuda()
    dy = (torch.randn(8, 512, 1024) * 0.05).bfloat16().cuda()
    # micro-batch j runs on stream j mod 2: the forward pass of a new micro-batch beside the backward pass of
    # the one in flight (schedule.MinibatchStreams; same results as one stream, bit for bit)
    rings = [schedule.MinibatchStreams(1) if overlap else None]
    if rings[0] is not None:
        rings[0].join()
    count = {"f": 0, "b": 0}
    pend = []

    def one_stream():
        if rings[0] is not None:
            rings[0].leave()
            rings[0] = None

    def forward():
        ring = rings[0]
        with (ring.forward(count["f"]) if ring is not None else contextlib.nullcontext()):
            pend.append(m(x))
        count["f"] += 1

    def step():
        forward()
        ring = rings[0]
        with (ring.backward(count["b"]) if ring is not None else contextlib.nullcontext()):
            opt.zero_grad()
            opt.load_old_params()
            pend.pop(0).backward(dy)
            opt.load_new_params()
            opt.step()
        count["b"] += 1

    forward()
    elapsed, stats = _run_steps(step, steps, warmup, one_stream)
    return elapsed, stats, 8, "bf16", ("PipeDream-2BW stage: 6 transformer layers (hidden 1024, 16 heads, FFN 4096, GELU, "
                                        "pre-LN), seq 512, micro-batch 8, 4-micro-batch accumulation, 2 weight versions, "
                                        "bf16 compute, fp32 master Adam"
                                        + (", forward of a new micro-batch beside the backward of the one in flight (one "
                                           "stream per micro-batch in flight)" if overlap else ", one stream"))


def gnmt_criterion_run(steps, warmup):
    """The tail of the last GNMT stage: classifier Linear(1024, 32320) + the label-smoothing criterion
    (smoothing 0.1, padding index 0, no padding rows) on [50, 128, 1024] activations, fp32, AdamWithWeightStashing with one
    version (the last stage keeps no stash).  One step = forward, loss, backward, update."""
    import torch
    from pipedream_amd import adam, layers
    torch.manual_seed(0)
    m = layers.Linear(1024, 32320).cuda()
    crit = layers.LabelSmoothing(0, 0.1)
    opt = adam.AdamWithWeightStashing([m], list(m.parameters()), None, 1.0, 1, lr=1e-3, betas=(0.9, 0.999))
    x = torch.randn(50, 128, 1024).cuda().requires_grad_(True)
    # no padding rows: the criterion kernels skip the logits of a padding row, which would flatter the
    # bytes-per-second figure computed from the full tensor size
    tgt = torch.randint(1, 32320, (50 * 128,)).cuda()

    def step():
        loss = crit(m(x), tgt)
        opt.zero_grad()
        opt.load_old_params()
        x.grad = None
        loss.backward()
        opt.load_new_params()
        opt.step()

    elapsed, stats = _run_steps(step, steps, warmup)
    return elapsed, stats, 128, "f32", ("GNMT classifier + label-smoothing criterion: Linear(1024, 32320) on seq 50 x batch 128, "
                                         "smoothing 0.1, no padding rows, fp32, Adam, 1 weight version")


def vgg16_pipeline_run(steps, warmup, stage_streams=True):
    """Full VGG16 (13 convolutions + 3 Linear layers) as the reference's four stages co-resident on the GPU,
    stash depths 4/3/2/1, batch 64 fp32, device-buffer hand-off, SGD momentum 0.9.  The pipeline is filled
    (3/2/1/0 forwards in flight), then one step = one minibatch through the steady state: every stage runs
    one forward, one backward and one stashed update, last stage first, so each stage finds its neighbour's
    gradient of the same minibatch and its producer's activation of the next one already queued.  Each stage
    launches on a stream of its own (the hand-off orders them with events), so kernels of different stages
    can share the GPU."""
    import torch
    from pipedream_amd import handoff, runtime, schedule, sgd
    from pipedream_amd.layers import CrossEntropyLoss
    from pipedream_amd.stages import vgg16
    handoff.reset_fabrics()
    torch.manual_seed(0)
    model = vgg16.model(CrossEntropyLoss(), dropout=0.5)
    conf = vgg16.conf()
    shapes = {"input0": (BATCH, 3, 224, 224), "target": (BATCH,)}
    dtypes = {"input0": torch.float32, "target": torch.int64}
    stages = []
    for rank in range(4):
        r = runtime.StageRuntime(
            model=model, distributed_backend="gloo", fp16=False, loss_scale=1.0,
            training_tensor_shapes=shapes, eval_tensor_shapes=dict(shapes), training_tensor_dtypes=dtypes,
            inputs_module_destinations={"input": 0}, target_tensor_names={"target"},
            configuration_maps={"module_to_stage_map": conf["module_to_stage_map"],
                                "stage_to_rank_map": conf["stage_to_rank_map"], "stage_to_depth_map": None},
            master_addr="127.0.0.1", rank=rank, local_rank=0, num_ranks_in_server=4, verbose_freq=0,
            model_type=runtime.IMAGE_CLASSIFICATION)
        opt = sgd.SGDWithWeightStashing(r.modules(), r.master_parameters, r.model_parameters, 1.0,
                                        num_versions=r.num_warmup_minibatches + 1, **SGD_KW)
        stages.append((r, opt))
    g = torch.Generator().manual_seed(0)
    images = [torch.randn(BATCH, 3, 224, 224, generator=g).cuda().contiguous(memory_format=torch.channels_last)
              for _ in range(2)]
    targets = [torch.randint(0, 1000, (BATCH,), generator=g).cuda() for _ in range(2)]

    def loader():
        i = 0
        while True:
            yield images[i % 2], targets[i % 2]
            i += 1

    total = warmup + steps + 4 + 3
    for i, (r, _) in enumerate(stages):
        r.train(total)
        r.set_loader(loader() if i == 0 else None)
    streams = schedule.stage_streams(4) if stage_streams else [torch.cuda.current_stream()] * 4
    torch.cuda.synchronize()
    for (r, _), stream in zip(stages, streams):          # fill: 3 / 2 / 1 / 0 forwards in flight
        with torch.cuda.stream(stream):
            for _ in range(r.num_warmup_minibatches):
                r.run_forward()

    def step():
        for (r, opt), stream in zip(reversed(stages), reversed(streams)):
            with torch.cuda.stream(stream):
                assert r.can_run_forward()
                r.run_forward()
                opt.zero_grad()
                opt.load_old_params()
                assert r.can_run_backward()
                r.run_backward()
                opt.load_new_params()
                opt.step()

    elapsed, stats = _run_steps(step, steps, warmup)
    done = warmup + steps + min(steps, 4)
    assert [o.latest_version.version for _, o in stages] == [done] * 4
    assert stages[0][1].queue.versions() == [done - 3 + i for i in range(4)]
    return elapsed, stats, BATCH, "f32", ("Full VGG16 as 4 co-resident stages (reference split conv1_1-conv1_2 / ..conv3_1 / "
                                           "..conv5_1 / rest + 3 FC), batch 64, fp32, stash depths 4/3/2/1, SGD momentum "
                                           "0.9, steady-state 1F1B, device-buffer hand-off")


# ---- CPU baselines of the other configurations: the oracle on a bounded sample ------------------------

def _time_cpu(step, timed, unit_per_step, sample):
    import torch
    step()
    t0 = time.perf_counter()
    for _ in range(timed):
        step()
    sec = (time.perf_counter() - t0) / timed
    return {"value": unit_per_step / sec, "unit": "samples/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": sample % {"timed": timed, "sec": sec}}


def cpu_vgg16_pipeline():
    """The oracle's 4-stage pipeline (torch.nn stages, state_dict-copy stashing, torch.optim.SGD) at batch 8:
    samples/s of a CPU convolution hardly depend on the batch size, and a batch-64 minibatch is 5.9 TFLOP."""
    import torch
    from oracle import models, pipeline_oracle, stash_oracle
    torch.manual_seed(0)
    batch, n = 16, 6
    stages = [models.VggStage0(), models.VggStage1(), models.VggStage2(), models.VggStage3(dropout=0.5)]
    g = torch.Generator().manual_seed(0)
    batches = [(torch.randn(batch, 3, 224, 224, generator=g), torch.randint(0, 1000, (batch,), generator=g))
               for _ in range(n)]
    t0 = time.perf_counter()
    pipeline_oracle.run_pipeline(stages, torch.nn.CrossEntropyLoss(),
                                 lambda s, m, nv: stash_oracle.StashingOptimizerOracle("SGD", [m], m.parameters(), nv, **SGD_KW),
                                 batches)
    sec = (time.perf_counter() - t0) / n
    return {"value": batch / sec, "unit": "samples/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": "%d minibatches of batch %d through the 4-stage oracle pipeline incl. fill and drain (%.1f s per "
                      "minibatch)" % (n, batch, sec)}


def cpu_gnmt():
    import torch
    from oracle import models, stash_oracle
    torch.manual_seed(0)
    m = models.GnmtStage0(dropout=0.0)
    opt = stash_oracle.StashingOptimizerOracle("Adam", [m], m.parameters(), 3, lr=1e-3, betas=(0.9, 0.999))
    ids = torch.randint(0, 32320, (50, 128))
    dy = torch.randn(50, 128, 1024) * 1e-2
    pend = [m(ids) for _ in range(2)]

    def step():
        pend.append(m(ids))
        opt.zero_grad()
        opt.load_old_params()
        pend.pop(0).backward(dy)
        opt.load_new_params()
        opt.step()

    return _time_cpu(step, 6, 128, "%(timed)d steady-state steps at seq 50 x batch 128 after 1 warm-up step (%(sec).1f s/step)")


def cpu_gnmt_criterion():
    import torch
    from oracle import seq2seq_oracle, stash_oracle
    torch.manual_seed(0)
    m = torch.nn.Linear(1024, 32320)
    opt = stash_oracle.StashingOptimizerOracle("Adam", [m], m.parameters(), 1, lr=1e-3, betas=(0.9, 0.999))
    x = torch.randn(50, 128, 1024, requires_grad=True)
    tgt = torch.randint(1, 32320, (50 * 128,))

    def step():
        loss = seq2seq_oracle.label_smoothing(m(x), tgt, 0, 0.1)
        opt.zero_grad()
        opt.load_old_params()
        x.grad = None
        loss.backward()
        opt.load_new_params()
        opt.step()

    return _time_cpu(step, 3, 128, "%(timed)d steps on seq 50 x batch 128 after 1 warm-up step (%(sec).1f s/step)")


def cpu_transformer():
    import torch
    from oracle import models, stash_oracle
    torch.manual_seed(0)
    m = models.TransformerStage0()
    opt = stash_oracle.StashingOptimizerOracle("Adam", [m], m.parameters(), 2, update_interval=4, lr=1e-3,
                                               betas=(0.9, 0.999))
    x = torch.randn(8, 512, 1024)
    dy = (torch.randn(8, 512, 1024) * 0.05).bfloat16()
    pend = [m(x)]

    def step():
        pend.append(m(x))
        opt.zero_grad()
        opt.load_old_params()
        pend.pop(0).backward(dy)
        opt.load_new_params()
        opt.step()

    return _time_cpu(step, 7, 8, "%(timed)d micro-batches of 8 x 512 tokens (two Adam updates among them) after 1 warm-up "
                                 "micro-batch (%(sec).1f s each), torch's bf16 CPU kernels")


CPU_BASELINES = {"vgg16_pipeline": cpu_vgg16_pipeline, "gnmt": cpu_gnmt, "gnmt_criterion": cpu_gnmt_criterion,
                 "transformer": cpu_transformer}


_SECONDARY = {"vgg16_pipeline": (vgg16_pipeline_run, "conv3x3_winograd_kernel", PEAK_FP32_MFMA_TFLOPS, "mfma"),
              "gnmt": (gnmt_run, "gemm_f32", PEAK_FP32_MFMA_TFLOPS, "mfma"),
              "gnmt_criterion": (gnmt_criterion_run, "label_smoothing_bwd", 8000.0, "hbm"),
              "transformer": (transformer_run, "gemm_bf16", 2500.0, "mfma")}


def secondary_record(workload, steps, warmup, single_stream=False, with_cpu_baseline=True, with_kernels=True):
    """One of the other configurations, measured like the headline one: the record of its line."""
    import gc
    import torch
    run, kernel, peak, bound = _SECONDARY[workload]
    if workload == "vgg16_pipeline":
        elapsed, stats, batch, dtype, desc = run(steps, warmup, stage_streams=not single_stream)
        desc += ", one stream for all stages" if single_stream else ", one stream per stage"
    elif workload in ("gnmt", "transformer"):
        elapsed, stats, batch, dtype, desc = run(steps, warmup, overlap=not single_stream)
    else:
        elapsed, stats, batch, dtype, desc = run(steps, warmup)
    gc.collect()
    torch.cuda.empty_cache()
    extra = {}
    total_us = lambda name: stats[name]["launches"] * stats[name]["avg_us"] if name in stats else 0.0
    if kernel == "gemm_f32" and total_us("gemm_f32_as_bf16x6") > total_us(kernel):
        # the large fp32 products run as six bf16 MFMA products of split operands: that launch (operand split,
        # bf16 GEMM over the six-fold reduction, and the sum of partial products where the output is narrow) is
        # the dominant one, measured against the bf16 MFMA peak with the flop it executes (6 x 2 M N K)
        kernel, peak = "gemm_f32_as_bf16x6", 2500.0
        k = dict(stats[kernel])
        extra = {"f32_equivalent": k["TFLOP/s"],
                 "note": "six bf16 MFMA products per fp32 product: executed flop = 6 x 2MNK; the launch time includes "
                         "the operand split (and the sum of partial products for narrow outputs)"}
        k["TFLOP/s"] = 6.0 * k["TFLOP/s"]
    else:
        k = dict(stats[kernel])
    if bound == "hbm":
        # the byte-moving kernels record algorithmic bytes as their work: the rate is in TB/s
        for name in ("label_smoothing_fwd", "label_smoothing_bwd"):
            stats[name]["GB/s"] = round(stats[name].pop("TFLOP/s") * 1e3, 1)
        k["TFLOP/s"] = stats[kernel]["GB/s"]
    if kernel == "conv3x3_winograd_kernel":
        # the Winograd kernel executes 16/36 of the direct convolution's multiplications
        extra = {"direct_equivalent": k["TFLOP/s"]}
        k["TFLOP/s"] = k["TFLOP/s"] * 16.0 / 36.0
    out = {
        "metric": "samples/sec per stage (fwd+bwd+stashed update)", "value": batch * steps / elapsed,
        "unit": "samples/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": 1e3 * elapsed / steps, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dtype, "data": "synthetic", "config": {"workload": desc, "global_batch": batch,
                                                        "parallelism": "1 stage on 1 GPU"},
        "roofline": {"bound": bound, "achieved": k["TFLOP/s"], "peak": peak,
                     "unit": "GB/s" if bound == "hbm" else "TFLOP/s",
                     "frac": k["TFLOP/s"] / peak, "traffic": None, "kernel": kernel, "launches": k["launches"],
                     "avg_us": k["avg_us"], **extra},
    }
    if workload in ("gnmt", "transformer") and not single_stream:
        # the timed steps run the passes of different minibatches side by side; the launch durations behind
        # the roofline come from instrumented steps on one stream, where a launch has the GPU to itself
        out["roofline"]["measured_on"] = "one stream (instrumented steps after the timed region)"
    if with_kernels:
        out["kernels"] = stats
    if workload in ("gnmt", "gnmt_criterion") and "gemm_f32_as_bf16x6" in stats:
        # Products of at least 2^32 multiply-adds with wide outputs (the LSTM input projections, the classifier's
        # forward and weight-gradient products) run as six bf16 MFMA products of three-way split fp32 operands
        # with fp32 accumulation (ops.set_gemm_f32_algorithm): closer to the fp64 product than the fp32 MFMA
        # kernel, and faster.  The same steps with every product on the fp32 MFMA kernels, for comparison:
        from pipedream_amd import ops
        out["config"]["workload"] += ("; fp32 products of at least 2^32 multiply-adds with at least 192 output tiles of "
                                      "256 x 256 computed as six bf16 MFMA products of three-way split operands, "
                                      "fp32 accumulation")
        out["dtype"] = "f32 (large products: 3 x bf16 split operands, f32 accumulation)"
        ops.set_gemm_f32_algorithm("mfma_f32")
        try:
            n = max(4, steps // 2)
            if workload == "gnmt":
                e2 = run(n, warmup, overlap=not single_stream)[0]
            else:
                e2 = run(n, warmup)[0]
        finally:
            ops.set_gemm_f32_algorithm("auto")
        gc.collect()
        torch.cuda.empty_cache()
        out["f32_mfma_only"] = {"ms_per_step": 1e3 * e2 / n, "value": batch * n / e2, "steps": n,
                                "note": "ops.set_gemm_f32_algorithm('mfma_f32'): every product on the fp32 MFMA kernels"}
    if with_cpu_baseline:
        out["cpu_baseline"] = CPU_BASELINES[workload]()
    return out


def secondary(args):
    print(json.dumps(secondary_record(args.workload, args.steps, args.warmup, args.single_stream,
                                      not args.no_cpu_baseline)))


# steps / warm-up steps of the other configurations inside the default run (each a few hundred milliseconds
# of GPU time; their CPU baselines are the bounded samples above, a few seconds each)
DEFAULT_RUN_WORKLOADS = {"vgg16_pipeline": (10, 3), "gnmt": (20, 5), "transformer": (40, 8)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--workload", default="vgg16_front", choices=["vgg16_front", "vgg16_pipeline", "gnmt", "gnmt_criterion", "transformer"],
                    help="vgg16_front (default) is the headline configuration; the others print the same kind of "
                         "line for the full VGG16 as four co-resident stages, the LSTM stage, the GNMT classifier + "
                         "criterion and the transformer stage")
    ap.add_argument("--single-stream", action="store_true",
                    help="vgg16_pipeline: launch all four stages on one stream instead of one stream per stage; "
                         "gnmt, transformer: forward and backward passes on one stream instead of one stream per minibatch in flight")
    ap.add_argument("--headline-only", action="store_true",
                    help="default workload: leave out the `workloads` object (the other configurations)")
    ap.add_argument("--pmc-probe", action="store_true",
                    help="run the counter-calibration copy and two benchmark steps, print no JSON")
    ap.add_argument("--traffic-bytes", type=float, default=None,
                    help="HBM bytes per launch of the dominant kernel from the PMC runs (see profiles/)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (one stage's share of the pipeline at its "
                 "real shape); --gpus %d is not supported" % args.gpus)
    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py: no HIP device; the product path has no CPU fallback")

    if args.pmc_probe:
        pmc_probe()
        return
    if args.workload != "vgg16_front":
        secondary(args)
        return
    elapsed, stats, _ = gpu_run(args.steps, args.warmup)
    wino = "conv3x3_winograd_kernel" in stats
    conv = stats["conv3x3_winograd_kernel" if wino else "conv3x3_fwd_kernel"]
    kernel = "winograd_fwd_kernel" if wino else "conv3x3_fwd_kernel"
    direct = conv["rate"] / 1e12
    # what the MFMA units execute: 16 multiplies per 2x2 outputs and channel pair instead of 36
    executed = direct * (16.0 / 36.0 if wino else 1.0)
    traffic = args.traffic_bytes if args.traffic_bytes is not None else measured_traffic(kernel)
    out = {
        "metric": "samples/sec per stage (fwd+bwd+stashed update), VGG16 bs64; optimizer HBM GB/s",
        "value": BATCH * args.steps / elapsed,
        "unit": "samples/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": 1e3 * elapsed / args.steps,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "VGG16 stage 0 (conv1_1..pool2), batch 64, fp32, stash depth 4, SGD momentum 0.9, "
                               "1F1B with 4 minibatches in flight",
                   "global_batch": BATCH, "parallelism": "1 stage on 1 GPU"},
        "roofline": {"bound": "mfma", "achieved": executed, "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
                     "frac": executed / PEAK_FP32_MFMA_TFLOPS, "traffic": traffic,
                     "kernel": kernel + (" (F(2x2,3x3); forward + input gradient)" if wino
                                         else "<.,.,16> (forward + input gradient)"),
                     "launches": conv["launches"], "avg_us": conv["avg_us"],
                     "flop_per_launch": conv["work_per_launch"] * (16.0 / 36.0 if wino else 1.0),
                     "direct_flop_per_launch": conv["work_per_launch"],
                     # the rate a direct convolution (2*9*C*K flop per output pixel) would need for this time
                     "direct_equivalent": direct},
        "kernels": {k: {"launches": v["launches"], "avg_us": round(v["avg_us"], 1),
                        "TFLOP/s": round(v["rate"] / 1e12, 2)} for k, v in stats.items()},
        "optimizer_hbm": optimizer_bandwidth("SGD"),
        "optimizer_hbm_adam": optimizer_bandwidth("Adam"),
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    if not args.headline_only:
        # the other configurations in the same record: throughput, dominant kernel against its roofline and
        # the CPU oracle's rate on a bounded sample, each measured after the headline's timed region
        import gc
        del stats
        gc.collect()
        torch.cuda.empty_cache()
        out["workloads"] = {name: secondary_record(name, steps, warmup, with_cpu_baseline=not args.no_cpu_baseline,
                                                   with_kernels=False)
                            for name, (steps, warmup) in DEFAULT_RUN_WORKLOADS.items()}
    print(json.dumps(out))


if __name__ == "__main__":
    main()

"""The 1F1B training loop of one stage, and a driver that interleaves the loops of
several co-resident stages on one GPU.

``stage_train_loop`` is the body of ``train()`` in the reference's caller
(runtime/image_classification/main_with_runtime.py:333-427): ``W`` warm-up forwards,
then ``n - W`` times [forward, adjust lr, zero_grad, load_old_params, backward,
load_new_params, step], then ``W`` times the backward half.  In the reference every
stage is its own process and simply blocks in a receive queue; here the loop is a
generator that yields whenever its next receive would find the queue empty, and
``run_pipeline`` round-robins the generators until all are finished.  ``stage_eval_loop`` is the
forward-only counterpart (``validate()``, main_with_runtime.py:429-487) with the ``ack`` clock.

Each loop can be given a stream of its own (``stream=``, or ``stage_streams(n)`` for one per stage):
everything the stage launches -- forward, backward, the stashed update -- then goes to that stream, the
hand-off layer orders the stages with events, and the HBM-bound kernels of one stage (pooling backward,
the optimizer, split-k reductions) can run beside the MFMA-bound kernels of another.  All streams have the
default priority.
"""
import contextlib

import torch


def stage_streams(num_stages):
    """One stream per co-resident stage (default priority)."""
    return [torch.cuda.Stream() for _ in range(num_stages)]


def _on(stream):
    return torch.cuda.stream(stream) if stream is not None else contextlib.nullcontext()


def _join(stream):
    """Start of a loop on a stream of its own: whatever the caller queued on its current stream before
    (the arena's initial copies and fills, ``module.cuda()``, loader tensors) is ordered before the
    stage's first kernel.  Side streams do not wait for the stream they were created on by themselves."""
    if stream is not None:
        stream.wait_stream(torch.cuda.current_stream())


def _leave(stream):
    """End of a loop: the caller's current stream waits for the stage's last kernel, so reading
    parameters, ``state_dict()`` or a checkpoint after the loop needs no host synchronisation."""
    if stream is not None:
        torch.cuda.current_stream().wait_stream(stream)


class MinibatchStreams(object):
    """Streams that let a stage's forward pass of one minibatch run beside the backward pass of an older one.

    In steady-state 1F1B a stage issues forward(k + W), backward(k), update(k), forward(k + W + 1), ...  The
    forward pass of minibatch k + W and the backward pass of minibatch k share no data (different activations,
    the newest weight version against a stashed one, and the update writes the ring's oldest slot, which neither
    reads), yet on one stream they run one after the other.  Here minibatch j does everything -- forward,
    backward, update -- on stream j mod (W + 1).  The forward pass of minibatch k + W + 1 needs the weights
    that update(k) wrote: same stream, ordered by itself.  The only order that crosses streams is
    update(k - 1) before backward(k) / update(k) (optimizer state and accumulated gradients), kept by one
    event.  Results are bit-identical to the single-stream order: the same kernels on the same operands.

    What it buys depends on the stage: kernels that fill the GPU by themselves (convolutions) gain nothing;
    the LSTM stage, whose recurrences are chains of short dependent launches, runs two chains side by side.

    Use: ``with ring.forward(j): ...`` around the forward pass of minibatch ``j``, ``with ring.backward(k): ...``
    around ``zero_grad`` .. ``step`` of minibatch ``k`` (``stage_train_loop(..., minibatch_streams=ring)`` does
    it), ``ring.join()`` before the first and ``ring.leave()`` after the last pass to order the ring against
    the caller's current stream.  All streams have the default priority."""

    def __init__(self, warmup):
        self.streams = [torch.cuda.Stream() for _ in range(int(warmup) + 1)]
        self._updated = None          # event behind the latest update
        # A parameter's gradient-accumulation node lives as long as any graph that reaches the parameter, i.e. for
        # ever under 1F1B, and stays on the stream of the first forward pass; the engine orders it against the
        # stream a later backward pass runs on by itself.  That is intended here, so its warning is switched off.
        quiet = getattr(torch.autograd.graph, "set_warn_on_accumulate_grad_stream_mismatch", None)
        if quiet is not None:
            quiet(False)

    def stream_of(self, minibatch):
        return self.streams[minibatch % len(self.streams)]

    def join(self):
        here = torch.cuda.current_stream()
        for s in self.streams:
            s.wait_stream(here)

    def leave(self):
        here = torch.cuda.current_stream()
        for s in self.streams:
            here.wait_stream(s)

    @contextlib.contextmanager
    def forward(self, minibatch):
        with torch.cuda.stream(self.stream_of(minibatch)):
            yield

    @contextlib.contextmanager
    def backward(self, minibatch):
        s = self.stream_of(minibatch)
        with torch.cuda.stream(s):
            if self._updated is not None:
                s.wait_event(self._updated)
            yield
            self._updated = torch.cuda.Event()
            self._updated.record(s)


def stage_train_loop(r, optimizer, num_minibatches, loader=None, lr_schedule=None, on_forward=None,
                     no_input_pipelining=False, stream=None, minibatch_streams=None):
    """Generator running one stage's 1F1B schedule.

    ``lr_schedule(step) -> lr`` is written into every param group each iteration, as
    ``adjust_learning_rate`` does (main_with_runtime.py:562-563).  ``on_forward(i, r)`` is
    called after each steady-state forward (where the reference reads ``r.loss``).  ``stream``: the
    stream this stage's kernels are launched on (default: torch's current stream); it is made current
    only around the stage's own calls, never across a ``yield``.  The stream is ordered behind the
    caller's current stream when the loop starts and the caller's current stream behind it when the
    loop ends.  ``minibatch_streams``: a ``MinibatchStreams(r.num_warmup_minibatches)`` instead of ``stream``;
    the forward pass of a new minibatch then runs beside the backward pass of the oldest one in flight."""
    n = num_minibatches
    if minibatch_streams is not None and stream is not None:
        raise ValueError("give either stream or minibatch_streams")
    ring = minibatch_streams
    if ring is not None:
        ring.join()
    _join(stream)
    r.train(n)
    r.set_loader(loader if (r.stage is None or r.stage == 0) else None)
    warmup = 0 if no_input_pipelining else min(r.num_warmup_minibatches, n)

    def forward():
        while not r.can_run_forward():
            yield r
        with (ring.forward(r.forward_minibatch_id) if ring is not None else _on(stream)):
            r.run_forward()

    def backward_and_update():
        while not r.can_run_backward():
            yield r
        with (ring.backward(r.backward_minibatch_id) if ring is not None else _on(stream)):
            optimizer.zero_grad()
            optimizer.load_old_params()
            r.run_backward()
            optimizer.load_new_params()
            optimizer.step()

    for _ in range(warmup):
        for blocked in forward():
            yield blocked
    for i in range(n - warmup):
        for blocked in forward():
            yield blocked
        if lr_schedule is not None:
            lr = lr_schedule(i)
            for param_group in optimizer.param_groups:
                param_group['lr'] = lr
        if on_forward is not None:
            with (ring.forward(r.forward_minibatch_id - 1) if ring is not None else _on(stream)):
                on_forward(i, r)
        for blocked in backward_and_update():
            yield blocked
    for _ in range(warmup):
        for blocked in backward_and_update():
            yield blocked
    r.wait()
    _leave(stream)
    if ring is not None:
        ring.leave()


def stage_eval_loop(r, num_minibatches, loader=None, on_forward=None, no_input_pipelining=False, stream=None):
    """Generator running one stage's forward-only schedule, the body of ``validate()`` in the
    reference's caller (runtime/image_classification/main_with_runtime.py:429-498): ``W`` warm-up
    forwards, then ``n - W`` times [forward, ack], then the ``W`` acknowledgements still outstanding
    (:497-498), so that every stage takes and passes on one ack per minibatch and no queue is left
    holding anything.  The ack is the clock: a stage takes its next
    steady-state minibatch only after its consumer has acknowledged the oldest outstanding one.
    Call it under ``torch.no_grad()`` as the reference does.  ``on_forward(i, r)`` is called after each
    steady-state forward (where the reference reads ``r.output`` / ``r.loss``)."""
    n = num_minibatches
    _join(stream)
    r.eval(n)
    r.set_loader(loader if (r.stage is None or r.stage == 0) else None)
    warmup = 0 if no_input_pipelining else min(r.num_warmup_minibatches, n)

    def ack():
        while not r.can_run_ack():
            yield r
        with _on(stream):
            r.run_ack()

    for i in range(n):
        while not r.can_run_forward():
            yield r
        with _on(stream):
            r.run_forward()
        if i < warmup:
            continue
        if on_forward is not None:
            with _on(stream):
                on_forward(i - warmup, r)
        for blocked in ack():
            yield blocked
    for _ in range(warmup):
        for blocked in ack():
            yield blocked
    r.wait()
    _leave(stream)


def run_pipeline(loops):
    """Drive the stage loops to completion.  ``loops`` are ``stage_train_loop``
    generators, first stage first.  A generator yields only when its stage is blocked on
    an empty queue; a full round in which every stage is blocked and none has advanced
    its minibatch counters is a deadlock and raises."""
    live = list(loops)
    last_signature = None
    while live:
        signature = []
        finished = False
        for g in list(live):
            try:
                r = next(g)
                signature.append((r.forward_minibatch_id, r.backward_minibatch_id))
            except StopIteration:
                live.remove(g)
                finished = True
        if live and not finished:
            if signature == last_signature:
                raise RuntimeError("pipeline schedule deadlocked: every stage waits for a tensor "
                                   "(minibatch counters %s)" % (signature,))
            last_signature = signature
        else:
            last_signature = None

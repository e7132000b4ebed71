"""Device-buffer hand-off of activations, gradients and acknowledgements between co-resident stages.

On one GPU the stages of a pipeline live in one process, so the transport of the reference's
``CommunicationHandler`` (helper threads + ``torch.distributed`` send/recv,
runtime/communication.py:610-712) collapses to passing the device tensor itself.  What is kept is
its queue contract (runtime/communication.py:583-608):

* one FIFO per tensor name, receiver and direction;
* a tensor received in the forward direction becomes a gradient-requiring leaf when it is fp32
  (:595-596);
* what is sent is detached from the sender's autograd graph (:699) -- without the copy, because
  neither side writes into a hand-off buffer afterwards;
* in a forward-only run an ``ack`` travels in the backward direction as the clock that keeps a stage
  from running ahead of its consumer (runtime/communication.py:193-211, runtime/runtime.py:629-653).

Added to it: every parcel carries the minibatch number it belongs to (the receiver checks that it
takes them in order) and a ``premasked`` flag, the producer's statement about who applies the backward
pass of the ReLU that ends the producing stage (see ``StageRuntime``).

Stages may run on streams of their own (``schedule.stage_train_loop(..., stream=...)``): whoever queues a
parcel records an event on the stream it is working on, whoever takes it makes its own stream wait for
that event (and tells the caching allocator that the tensor is now in use there), so a consumer's kernels
never start before the producer's have finished, whatever order the host issued them in.  On a single
stream the wait is a no-op.
"""
import collections

import torch

ACK = "ack"

Parcel = collections.namedtuple("Parcel", "tensor seq premasked ready")


class HandoffContractError(RuntimeError):
    """Producer and consumer of a hand-off disagree about the gradient they exchange."""


def becomes_leaf(tensor):
    """A received tensor of this kind takes part in the consumer's backward pass and gets a gradient
    sent back (runtime/communication.py:595)."""
    return torch.is_tensor(tensor) and tensor.dtype == torch.float32


class HandoffFabric(object):
    """The queues shared by the stages of one pipeline."""

    def __init__(self):
        self.queues = collections.defaultdict(collections.deque)
        self.bytes_sent = 0

    def queue(self, tensor_name, receiver_rank, backward):
        return self.queues[(tensor_name, receiver_rank, bool(backward))]

    def put(self, tensor_name, receiver_rank, backward, tensor, seq=None, premasked=False):
        """Queue ``tensor`` for ``receiver_rank``; also the way a test or a benchmark plays a neighbour
        stage that is not there."""
        self.bytes_sent += tensor.element_size() * tensor.nelement()
        ready = None
        if tensor.is_cuda:
            ready = torch.cuda.Event()
            ready.record()            # on the producer's current stream, behind the kernels that wrote the tensor
        self.queue(tensor_name, receiver_rank, backward).append(Parcel(tensor.detach(), seq, bool(premasked), ready))

    def take(self, tensor_name, receiver_rank, backward):
        """The oldest parcel queued for ``receiver_rank``, safe to use on the caller's current stream."""
        parcel = self.queue(tensor_name, receiver_rank, backward).popleft()
        if parcel.ready is not None:
            stream = torch.cuda.current_stream()
            stream.wait_event(parcel.ready)
            parcel.tensor.record_stream(stream)
        return parcel


_FABRICS = {}


def fabric_for(key):
    """Stages created with the same key (``(master_addr, master_port)``) share a fabric."""
    if key not in _FABRICS:
        _FABRICS[key] = HandoffFabric()
    return _FABRICS[key]


def reset_fabrics():
    _FABRICS.clear()


class DeviceHandoff(object):
    """One stage's end of the fabric.  ``inbound`` / ``outbound`` map a tensor name to the rank it comes
    from / goes to in the forward direction; gradients and acknowledgements take the same routes
    backwards."""

    def __init__(self, fabric_key, rank, inbound, outbound, ack_to=None):
        self.rank = rank
        self.fabric = fabric_for(fabric_key)
        self.inbound = dict(inbound)
        self.outbound = dict(outbound)
        self.forward_only = False
        self._ack = None
        self._ack_to = ack_to          # rank of the previous stage, None for the first

    def begin_run(self, forward_only):
        """Start of a ``train`` / ``eval`` run.  Whatever still waits for this stage in the backward
        direction is left over from an earlier run (its senders act only on what this stage hands them in
        the current one) and is dropped; the forward direction may already hold the first minibatches of
        an upstream stage that started earlier and is kept."""
        self.forward_only = forward_only
        for (name, receiver, backward), q in self.fabric.queues.items():
            if receiver == self.rank and backward:
                q.clear()

    def wait(self):
        """The reference joins its helper threads here (runtime/communication.py:357-367); device
        tensors handed over in-process are complete when queued."""

    def ready(self, names, backward):
        return all(len(self.fabric.queue(n, self.rank, backward)) > 0 for n in names)

    def take(self, tensor_name, seq, backward):
        q = self.fabric.queue(tensor_name, self.rank, backward)
        if not q:
            raise RuntimeError(
                "stage rank %s: nothing queued for %r (%s); the schedule ran this stage before its "
                "neighbour produced the tensor" % (self.rank, tensor_name, "backward" if backward else "forward"))
        parcel = self.fabric.take(tensor_name, self.rank, backward)
        if parcel.seq is not None and parcel.seq != seq:
            raise RuntimeError("stage rank %s: %r of minibatch %s arrived where minibatch %s was due"
                               % (self.rank, tensor_name, parcel.seq, seq))
        if not backward and becomes_leaf(parcel.tensor):
            parcel = parcel._replace(tensor=parcel.tensor.requires_grad_())
        return parcel

    def put(self, tensor_name, tensor, seq, backward, premasked=False):
        receiver = self.inbound[tensor_name] if backward else self.outbound[tensor_name]
        self.fabric.put(tensor_name, receiver, backward, tensor, seq, premasked)

    def put_ack(self, seq):
        if self._ack is None:
            self._ack = torch.zeros(1, dtype=torch.int64, device="cuda")
        self.fabric.put(ACK, self._ack_to, True, self._ack, seq)

"""Device-buffer hand-off of activations and gradients between co-resident stages.

On one GPU the stages of a pipeline live in one process, so the transport of the
reference's ``CommunicationHandler`` (helper threads + ``torch.distributed`` send/recv,
runtime/communication.py:610-712) collapses to passing the device tensor itself.  What
is kept is its queue contract (runtime/communication.py:583-608):

* one FIFO per tensor name, receiver and direction;
* a tensor received in the forward direction becomes a gradient-requiring leaf when it
  is fp32 (:595-596);
* what is sent is detached from the sender's autograd graph (:699) -- without the copy,
  because neither side writes into a hand-off buffer afterwards.

All stages launch on torch's current stream, so queue order is execution order and no
events are needed.
"""
import collections


class HandoffFabric(object):
    """The queues shared by the stages of one pipeline."""

    def __init__(self):
        self.queues = collections.defaultdict(collections.deque)
        self.bytes_sent = 0

    def queue(self, tensor_name, receiver_rank, backward):
        return self.queues[(tensor_name, receiver_rank, bool(backward))]


_FABRICS = {}


def fabric_for(key):
    """Stages created with the same ``(master_addr, master_port)`` share a fabric."""
    if key not in _FABRICS:
        _FABRICS[key] = HandoffFabric()
    return _FABRICS[key]


def reset_fabrics():
    _FABRICS.clear()


class DeviceHandoff(object):
    """Per-stage endpoint with the ``recv`` / ``send`` signature of the reference's
    ``CommunicationHandler`` (runtime/communication.py:583-608)."""

    def __init__(self, master_addr, master_port, rank, local_rank, num_ranks_in_server, world_size, fp16,
                 backend):
        self.rank = rank
        self.local_rank = local_rank
        self.world_size = world_size
        self.backend = backend
        self.fabric = fabric_for((master_addr, master_port))

    def initialize(self, receive_ranks, send_ranks, tensor_tags, target_tensor_names, training_tensor_dtypes,
                   rank_in_stage, num_ranks_in_stage, ranks_in_previous_stage, ranks_in_next_stage):
        self.receive_ranks = receive_ranks
        self.send_ranks = send_ranks
        self.tensor_tags = tensor_tags
        self.target_tensor_names = target_tensor_names
        self.training_tensor_dtypes = training_tensor_dtypes
        self.rank_in_stage = rank_in_stage
        self.num_ranks_in_stage = num_ranks_in_stage
        self.ranks_in_previous_stage = ranks_in_previous_stage
        self.ranks_in_next_stage = ranks_in_next_stage
        # Targets travel with the activations from stage to stage; the reference adds them
        # to the (shared) rank tables here too (runtime/communication.py:165-200).
        for name in target_tensor_names:
            if len(ranks_in_previous_stage) > 0:
                receive_ranks[name] = ranks_in_previous_stage
            if len(ranks_in_next_stage) > 0:
                send_ranks[name] = ranks_in_next_stage
        for name, ranks in list(receive_ranks.items()) + list(send_ranks.items()):
            if len(ranks) != 1:
                raise NotImplementedError(
                    "tensor %r is exchanged with %d ranks; replicated stages need more than one GPU"
                    % (name, len(ranks)))

    # helper threads do not exist here; the calls are kept so callers need not change
    def set_tensor_shapes(self, tensor_shapes):
        self.tensor_shapes = tensor_shapes

    def start_helper_threads(self, num_iterations, forward_only):
        self.forward_only = forward_only

    def increment_messaging_index(self, sending):
        pass

    def wait(self):
        pass

    # ---------------------------------------------------------------------------------
    def _recv_queue(self, tensor_name, backward):
        return self.fabric.queue(tensor_name, self.rank, backward)

    def can_recv(self, tensor_name, backward=False):
        return len(self._recv_queue(tensor_name, backward)) > 0

    def recv(self, tensor_name, forward_minibatch_id, backward_minibatch_id, backward=False):
        q = self._recv_queue(tensor_name, backward)
        if not q:
            raise RuntimeError(
                "stage rank %s: nothing queued for %r (%s); the schedule ran this stage before its "
                "neighbour produced the tensor" % (self.rank, tensor_name, "backward" if backward else "forward"))
        tensor = q.popleft()
        if not backward:
            import torch
            if tensor.dtype == torch.float32:
                tensor = tensor.requires_grad_()
        return tensor

    def send(self, tensor_name, tensor, forward_minibatch_id, backward_minibatch_id, backward=False):
        if backward:
            dst = self.receive_ranks[tensor_name][0]
        else:
            dst = self.send_ranks[tensor_name][0]
        self.fabric.bytes_sent += tensor.element_size() * tensor.nelement()
        self.fabric.queue(tensor_name, dst, backward).append(tensor.detach())

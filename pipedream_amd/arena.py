"""Flat-buffer weight-version ring in HBM.

One contiguous device buffer holds ``num_versions`` slots; every stashable state entry
of the stage's modules (parameters and buffers) has a fixed byte offset inside a slot.
The live module tensors are *views* into whichever slot is loaded, so
``load_old_params`` / ``load_new_params`` are pointer swaps (``tensor.data = view``) and
move no bytes.  Which slot holds which version is decided by the integer-only ring in
the C library (``pd_ring_*``).

Restates the storage side of ``OptimizerWithWeightStashing`` in the reference:
runtime/optimizer.py:58-62 (``initialize_queue`` clones the state ``num_versions``
times), :64-85 (``get_params``: ``running_*`` keys are never stashed, ``mask`` keys are
not rolled back), :87-116 (``set_params`` / ``load_old_params`` / ``load_new_params``).
"""
import collections
import ctypes

import torch

from . import _cabi

ALIGN = 256  # bytes; every entry and every slot starts on a 256-byte boundary


STAGGER = 4096            # bytes between the start addresses of operand streams, modulo STAGGER_PERIOD
STAGGER_PERIOD = 16384
# Entries of at least BIG_ENTRY bytes start BIG_ENTRY_PHASE bytes past a STAGGER boundary of their slot: their
# gradients come from the allocator on large power-of-two boundaries, and with the parameter streams a quarter
# of a 4 KiB granule off that grid the fused step measured 0.81 (SGD) / 0.78 (Adam) of the HBM peak on VGG16's
# 32 tensors instead of 0.78 / 0.72 with entries packed at 256-byte granularity.
BIG_ENTRY = 1 << 20
BIG_ENTRY_PHASE = 1024


def _round_up(x, a):
    return (x + a - 1) // a * a


def staggered_empty(nbytes, device, position):
    """A uint8 device buffer of ``nbytes`` whose start address is ``position * STAGGER`` modulo
    ``STAGGER_PERIOD``.  Returns (the allocation that owns the memory, the buffer as a view of it)."""
    raw = torch.empty(nbytes + STAGGER_PERIOD, dtype=torch.uint8, device=device)
    shift = (position * STAGGER - raw.data_ptr()) % STAGGER_PERIOD
    buf = raw[shift:shift + nbytes]
    if buf.data_ptr() % ALIGN:
        raise RuntimeError("allocator returned a buffer that is not %d-byte aligned" % ALIGN)
    return raw, buf


def _stashable(key):
    # optimizer.py:76-78 and :93-94: running statistics accumulate normally and masks
    # are taken from the live module, so neither is ever rolled back.
    return "running_" not in key and "mask" not in key


class Entry(object):
    __slots__ = ("tensor", "keys", "offset", "nbytes", "numel", "dtype", "shape", "stride",
                 "master_index", "views")

    def __init__(self, tensor):
        self.tensor = tensor
        self.keys = []          # [(module index, state_dict key)]
        self.offset = 0
        self.numel = tensor.numel()
        self.nbytes = tensor.numel() * tensor.element_size()
        self.dtype = tensor.dtype
        self.shape = tuple(tensor.shape)
        self.stride = tuple(tensor.stride())
        self.master_index = None
        self.views = []         # one view per physical slot


def _is_dense(t):
    if t.is_contiguous():
        return True
    # dense, non-overlapping in some permutation (e.g. channels_last)
    pairs = sorted((st, sz) for st, sz in zip(t.stride(), t.shape) if sz > 1)
    expect = 1
    for st, sz in pairs:
        if st != expect:
            return False
        expect *= sz
    return True


class WeightArena(object):
    """``num_versions`` flat slots + the integer ring that orders them."""

    def __init__(self, modules, master_parameters, num_versions, bf16_image=False, model_parameters=None):
        """``model_parameters`` (16-bit tensors, the modules' own parameters, one per master in the same order):
        the mixed-precision arrangement of runtime/optimizer.py:137-155.  The ring then stashes the 16-bit
        model parameters (they are what forward and backward passes read), ``master_parameters`` stay
        separate fp32 tensors outside the ring, and the fused step updates a master in place while it
        writes its 16-bit image into the ring's write slot."""
        self._lib = _cabi.lib()
        self.modules = list(modules)
        self.num_versions = int(num_versions)
        if self.num_versions < 1:
            raise ValueError("num_versions must be >= 1")

        masters = list(master_parameters)
        if not masters:
            raise ValueError("optimizer got an empty parameter list")
        device = masters[0].device
        _cabi.require_device(masters[0], "master parameter")
        self.fp32_masters = None
        self.half_dtype = None
        if model_parameters is not None:
            model_parameters = list(model_parameters)
            if bf16_image:
                raise ValueError("bf16_image keeps a 16-bit copy of fp32 module parameters; with model_parameters "
                                 "the module parameters are the 16-bit copy")
            if len(model_parameters) != len(masters):
                raise ValueError("model_parameters and master_parameters differ in length")
            self.half_dtype = model_parameters[0].dtype
            if self.half_dtype not in (torch.bfloat16, torch.float16):
                raise TypeError("model parameters must be bfloat16 or float16, got %s" % self.half_dtype)
            for q, p in zip(model_parameters, masters):
                if q.dtype != self.half_dtype or p.dtype != torch.float32 or q.shape != p.shape or q.device != device:
                    raise TypeError("every model parameter must be a %s tensor with an fp32 master of its shape on %s"
                                    % (self.half_dtype, device))
                if not p.is_contiguous() or p.data_ptr() % 16:
                    raise ValueError("fp32 masters must be contiguous, 16-byte aligned tensors")
            self.fp32_masters = masters
            masters = model_parameters          # what the ring stashes

        by_id = collections.OrderedDict()
        # 1. master parameters first, in optimizer order: they form one fp32 section that
        #    the fused step kernel walks.
        for i, p in enumerate(masters):
            if p.dtype != (self.half_dtype or torch.float32):
                raise TypeError("master parameters must be fp32, got %s" % p.dtype)
            if p.device != device:
                raise ValueError("all parameters of a stage must live on one device")
            if id(p) in by_id:
                raise ValueError("duplicate parameter in master_parameters")
            e = Entry(p)
            e.master_index = i
            by_id[id(p)] = e
        self.num_master = len(masters)

        # 2. every other stashable state entry of the modules (buffers, frozen params).
        for mi, module in enumerate(self.modules):
            owners = dict(module.named_parameters(remove_duplicate=False))
            owners.update(dict(module.named_buffers(remove_duplicate=False)))
            for key in module.state_dict().keys():
                t = owners.get(key)
                if t is None or not _stashable(key):
                    continue
                if t.device != device:
                    raise ValueError("state entry %r is on %s, expected %s" % (key, t.device, device))
                e = by_id.get(id(t))
                if e is None:
                    e = Entry(t)
                    by_id[id(t)] = e
                e.keys.append((mi, key))
        self.entries = list(by_id.values())

        off = 0
        for e in self.entries:
            if not _is_dense(e.tensor):
                # strided views cannot be re-homed; make the owner dense first
                e.tensor.data = e.tensor.data.contiguous()
                e.stride = tuple(e.tensor.stride())
            if e.nbytes >= BIG_ENTRY:
                off = _round_up(off - BIG_ENTRY_PHASE, STAGGER) + BIG_ENTRY_PHASE
            e.offset = off
            off = _round_up(off + e.nbytes, ALIGN)
            if e.master_index == self.num_master - 1:
                self.master_bytes = off
        self.other_bytes = max(off, ALIGN) - self.master_bytes
        # The fused step streams a slot it reads, a slot it writes, the gradients and the optimizer state at
        # the same element offset.  HBM bandwidth drops by 5-8 % when those streams start at the same address
        # modulo 16 KiB, so consecutive slots are staggered by 4 KiB (and the optimizer's flat state buffers,
        # ``staggered_empty`` in fused_optim, by 8 and 12 KiB).
        self.slot_bytes = _round_up(max(off, ALIGN), STAGGER_PERIOD) + STAGGER
        self._raw_buffer, self.buffer = staggered_empty(self.num_versions * self.slot_bytes, device, 0)
        # padding between entries must stay finite: the fused step walks it too
        self._lib.pd_fill_zero(ctypes.c_void_p(self.buffer.data_ptr()), self.buffer.numel(), _cabi.stream_ptr())

        handle = ctypes.c_void_p()
        self._lib.pd_ring_create(ctypes.c_void_p(self.buffer.data_ptr()), self.slot_bytes, self.num_versions,
                                 ctypes.byref(handle))
        self._ring = handle

        # Entries the optimizer does not own (buffers such as num_batches_tracked, frozen
        # parameters) keep the reference's copy semantics: the live module holds its own
        # copy, so what a forward pass writes into it does not leak into a stashed version.
        # They live together in one flat "live" block so a load/store is a single copy.
        self.live_other = torch.empty(max(self.other_bytes, ALIGN), dtype=torch.uint8, device=device)

        def _view(buf, lo, e):
            flat = buf[lo:lo + e.nbytes].view(e.dtype)
            if e.tensor.is_contiguous():
                return flat.view(e.shape)
            return flat.as_strided(e.shape, e.stride)

        for e in self.entries:
            for s in range(self.num_versions):
                e.views.append(_view(self.buffer, s * self.slot_bytes + e.offset, e))
        self.masters = self.entries[:self.num_master]
        self.others = self.entries[self.num_master:]

        # initial state: newest entry (queue[-1]) holds the live values, then clone it
        # into every other slot (optimizer.py:58-62).
        self.live_slot = self.entry(-1)[0]
        with torch.no_grad():
            for e in self.entries:
                e.views[self.live_slot].copy_(e.tensor.detach())
            for e in self.others:
                live = _view(self.live_other, e.offset - self.master_bytes, e)
                live.copy_(e.tensor.detach())
                e.tensor.data = live
        self._lib.pd_ring_broadcast(self._ring, self.live_slot, self.slot_bytes, _cabi.stream_ptr())
        self._point_live_at(self.live_slot)

        # Optional bf16 image of the master section, one per slot, with the same element
        # offsets: what bf16-compute layers multiply with.  The fused optimizer step keeps
        # it current (it writes the bf16 value next to every fp32 parameter it produces).
        self.bf16_image = None
        if bf16_image:
            n = self.master_bytes // 4
            self.bf16_image = [torch.empty(n, dtype=torch.bfloat16, device=device) for _ in range(self.num_versions)]
            for s in range(self.num_versions):
                self._lib.pd_cast_f32_to_bf16(ctypes.c_void_p(self.slot_ptr(s)),
                                              ctypes.c_void_p(self.bf16_image[s].data_ptr()), n, _cabi.stream_ptr())
            for e in self.masters:
                lo = e.offset // 4
                views = []
                for s in range(self.num_versions):
                    flat = self.bf16_image[s][lo:lo + e.numel]
                    views.append(flat.view(e.shape) if e.tensor.is_contiguous() else flat.as_strided(e.shape, e.stride))
                # layers look these up through the parameter object
                e.tensor._pd_bf16_views = views
                e.tensor._pd_arena = self

    def __del__(self):
        ring = getattr(self, "_ring", None)
        if ring is not None and ring.value:
            try:
                self._lib.pd_ring_destroy(ring)
            except Exception:
                pass
            self._ring = None

    # -- ring bookkeeping (host integers) ------------------------------------------
    def entry(self, queue_index):
        """(physical slot, version) of ``queue[queue_index]``; index 0 is the oldest."""
        slot = ctypes.c_int()
        version = ctypes.c_int64()
        self._lib.pd_ring_entry(self._ring, int(queue_index), ctypes.byref(slot), ctypes.byref(version))
        return slot.value, version.value

    def write_slot(self):
        slot = ctypes.c_int()
        self._lib.pd_ring_write_slot(self._ring, ctypes.byref(slot))
        return slot.value

    def push(self, version):
        slot = ctypes.c_int()
        self._lib.pd_ring_push(self._ring, int(version), ctypes.byref(slot))
        return slot.value

    def slot_ptr(self, slot):
        return self.buffer.data_ptr() + slot * self.slot_bytes

    # -- live pointers -------------------------------------------------------------
    def _point_live_at(self, slot):
        for e in self.masters:
            e.tensor.data = e.views[slot]
        self.live_slot = slot

    def load_slot(self, slot, with_others=True):
        """Make the parameters views of ``slot`` (no bytes move) and, as the reference's
        ``set_params`` does, overwrite the live copy of the remaining entries."""
        if slot != self.live_slot:
            self._point_live_at(slot)
        if with_others and self.other_bytes:
            self._lib.pd_copy(ctypes.c_void_p(self.live_other.data_ptr()),
                              ctypes.c_void_p(self.slot_ptr(slot) + self.master_bytes),
                              self.other_bytes, _cabi.stream_ptr())

    def store_others(self, dst_slot, stream=None):
        """Live copy of the non-optimised entries -> ``dst_slot`` (the part of
        ``get_params(clone=False)`` the fused step does not cover)."""
        if self.other_bytes:
            self._lib.pd_copy(ctypes.c_void_p(self.slot_ptr(dst_slot) + self.master_bytes),
                              ctypes.c_void_p(self.live_other.data_ptr()),
                              self.other_bytes, _cabi.stream_ptr(stream))

    def copy_masters(self, src_slot, dst_slot, stream=None):
        if src_slot == dst_slot or self.master_bytes == 0:
            return
        self._lib.pd_copy(ctypes.c_void_p(self.slot_ptr(dst_slot)), ctypes.c_void_p(self.slot_ptr(src_slot)),
                          self.master_bytes, _cabi.stream_ptr(stream))

    def refresh_bf16_image(self, slot=None):
        """Re-cast the bf16 image of ``slot`` (default: the loaded one) from its fp32 masters.  The fused
        optimizer step keeps the image current by itself; this is for the writes that bypass it (a foreign
        ``state_dict`` copied into the parameters, ``get_params(clone=False)``, an in-place edit by the
        caller)."""
        if self.bf16_image is None:
            return
        slot = self.live_slot if slot is None else slot
        self._lib.pd_cast_f32_to_bf16(ctypes.c_void_p(self.slot_ptr(slot)),
                                      ctypes.c_void_p(self.bf16_image[slot].data_ptr()), self.master_bytes // 4,
                                      _cabi.stream_ptr())

    def master_view(self, master_index, slot):
        return self.entries[master_index].views[slot]

    def state_dicts(self, slot):
        """Per-module OrderedDicts of views into ``slot`` (the reference's stash format)."""
        dicts = [collections.OrderedDict() for _ in self.modules]
        for e in self.entries:
            for (mi, key) in e.keys:
                dicts[mi][key] = e.views[slot]
        for d in dicts:
            d._pd_slot = slot
        return dicts

"""Host-side mirror of the reference's CMS timing and optimizer types
(core/src/conductor.rs, core/src/adamw.rs, core/src/gpu_optimizer.rs) over the
C ABI.  Same names and semantics: `Conductor.pulse()` does not advance;
`advance()` is called after every observer has read the pulse."""
import ctypes
from dataclasses import dataclass
from typing import List

from .ffi import lib


@dataclass
class Pulse:
    """core/src/conductor.rs:12-17."""
    global_step: int
    active_levels: List[bool]

    def bitmask(self) -> int:
        """core/src/gpu_forward.rs:2449 pulse_to_bitmask."""
        k = len(self.active_levels)
        arr = (ctypes.c_int * k)(*[int(a) for a in self.active_levels])
        return lib.nlh_pulse_to_bitmask(arr, k)


class RestoreError(Exception):
    pass


class Conductor:
    """core/src/conductor.rs:36-155."""

    def __init__(self, k, chunk_sizes):
        assert len(chunk_sizes) == k, "chunk_sizes length must equal k"
        assert k >= 1, "k must be at least 1"
        for i, cs in enumerate(chunk_sizes):
            assert cs >= 1, f"chunk_sizes[{i}] must be >= 1"
        self.k = k
        self.chunk_sizes = list(chunk_sizes)
        arr = (ctypes.c_longlong * k)(*chunk_sizes)
        self._h = lib.nlh_conductor_new(k, arr)
        if not self._h:
            raise ValueError("nlh_conductor_new failed")

    def __del__(self):
        if getattr(self, "_h", None):
            lib.nlh_conductor_free(self._h)
            self._h = None

    def set_seq_len(self, seq_len):
        lib.nlh_conductor_set_seq_len(self._h, seq_len)

    def pulse(self) -> Pulse:
        act = (ctypes.c_int * self.k)()
        lib.nlh_conductor_pulse(self._h, act)
        return Pulse(self.step(), [bool(a) for a in act])

    def advance(self):
        lib.nlh_conductor_advance(self._h)

    def step(self) -> int:
        return lib.nlh_conductor_step(self._h)

    def restore(self, k, chunk_sizes, step, stream_pulse_id):
        arr = (ctypes.c_longlong * len(chunk_sizes))(*chunk_sizes)
        rc = lib.nlh_conductor_restore(self._h, k, arr, step, stream_pulse_id)
        if rc == 1:
            raise RestoreError("ConfigMismatch")
        if rc == 2:
            raise RestoreError("PulseMismatch")


class FrequencyAwareAdamW:
    """core/src/adamw.rs FrequencyAwareAdamW / core/src/gpu_optimizer.rs:403 gpu_adamw_update:
    always-active tensors (group -1) and per-level tensors gated by the Pulse."""

    def __init__(self, k, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.01):
        self.k = k
        self._h = lib.nlh_adamw_new(k, beta1, beta2, eps, weight_decay)
        self._keep = []

    def __del__(self):
        if getattr(self, "_h", None):
            lib.nlh_adamw_free(self._h)
            self._h = None

    def add_tensor(self, group, w, g, m, v):
        for t in (w, g, m, v):
            assert t.is_cuda and t.is_contiguous() and t.numel() == w.numel()
        self._keep.append((w, g, m, v))
        return lib.nlh_adamw_add_tensor(self._h, group, w.data_ptr(), g.data_ptr(), m.data_ptr(),
                                        v.data_ptr(), w.numel())

    def set_clamp(self, tensor_id, lo, hi):
        lib.nlh_adamw_set_clamp(self._h, tensor_id, lo, hi)

    def step(self, pulse: Pulse, lr, max_grad_norm=0.0, norm_scale=None):
        act = (ctypes.c_int * self.k)(*[int(a) for a in pulse.active_levels[:self.k]])
        rc = lib.nlh_adamw_step(self._h, act, lr, max_grad_norm,
                                norm_scale.data_ptr() if norm_scale is not None else None)
        if rc:
            raise RuntimeError(f"nlh_adamw_step failed ({rc})")

    def swa_step(self):
        return lib.nlh_adamw_swa_step(self._h)

    def level_step(self, level):
        return lib.nlh_adamw_level_step(self._h, level)


def _ptr_array(tensors):
    return (ctypes.c_void_p * len(tensors))(*[t.data_ptr() for t in tensors])


class ErrorBuffer:
    """core/src/conductor.rs:224-261: outer-loop gradients a frozen level receives are summed here and
    applied as one plain gradient step when the level fires.  `like` is the level's parameter tensors
    (device, float32): one accumulator of the same size is kept per tensor, in the same order."""

    def __init__(self, like):
        import torch
        self.grads = [torch.zeros_like(t) for t in like]
        self._h = lib.nlh_error_buffer_new()
        for g in self.grads:
            assert g.is_cuda and g.is_contiguous() and g.dtype == torch.float32
            lib.nlh_error_buffer_add_tensor(self._h, g.data_ptr(), g.numel())

    def __del__(self):
        if getattr(self, "_h", None):
            lib.nlh_error_buffer_free(self._h)
            self._h = None

    @property
    def steps_accumulated(self) -> int:
        return lib.nlh_error_buffer_steps(self._h)

    def _check(self, tensors):
        assert len(tensors) == len(self.grads)
        for t, g in zip(tensors, self.grads):
            assert t.is_cuda and t.is_contiguous() and t.numel() == g.numel()

    def accumulate(self, level_grads):
        self._check(level_grads)
        lib.nlh_error_buffer_accumulate(self._h, _ptr_array(level_grads))

    def apply_and_reset(self, params, lr):
        self._check(params)
        lib.nlh_error_buffer_apply_and_reset(self._h, _ptr_array(params), lr)

    def health_check(self, single_step_grads):
        """-> ||accumulated|| / ||single_step||, or None when the single-step norm is below 1e-12."""
        self._check(single_step_grads)
        ratio = ctypes.c_float(0.0)
        rc = lib.nlh_error_buffer_health_check(self._h, _ptr_array(single_step_grads), ctypes.byref(ratio))
        if rc < 0:
            raise RuntimeError("nlh_error_buffer_health_check failed")
        return ratio.value if rc == 1 else None


class ContextState:
    """core/src/conductor.rs:156-221: the memories that persist across forward calls.  `memory[l]` is
    level l's state ([chains, d, d] here: one matrix per batch element and head), `momentum[l]` the Titans
    momentum carried with it, `self_ref[l]` a [chains, 6, d, d] block of self-referential memories
    (m_k, m_v, m_q, m_eta, m_alpha, m_mem) or None when the projections are static."""

    def __init__(self, memory, momentum=None, self_ref=None):
        self.memory = list(memory)
        self.momentum = list(momentum) if momentum is not None else []
        self.self_ref = list(self_ref) if self_ref is not None else [None] * len(self.memory)

    def reset(self):
        """:212-219: zero every memory in place (document boundary); the Conductor's step is untouched."""
        bufs = [t for t in self.memory + self.momentum + self.self_ref if t is not None]
        if bufs:
            n = (ctypes.c_int * len(bufs))(*[t.numel() for t in bufs])
            lib.nlh_context_state_reset(_ptr_array(bufs), n, len(bufs))

    def seed_self_ref(self, level_inits):
        """:193-206: level_inits[l] = dict with m_k_init, m_v_init, m_q_init, m_eta_init, m_alpha_init
        ([d, d] tensors, or absent for static projections) and m_mem_init (or absent).  Per level, as there: the five
        projection memories are seeded when m_k_init is given (a level without a self-referential block is skipped,
        later levels are still visited); m_mem_init, when its size matches, is copied into memory[l] whether or not
        the projections are static (every chain of the level starts from it), and into slot 5 of the level's
        self-referential block, which is the copy the HOPE kernels read."""
        for lv, init in enumerate(level_inits):
            if lv >= len(self.self_ref):
                break
            mems = self.self_ref[lv]
            get = lambda n: init[n].data_ptr() if init.get(n) is not None else None
            mm = init.get("m_mem_init")
            if mems is not None and init.get("m_k_init") is not None:
                chains, six, d, _ = mems.shape
                assert six == 6
                lib.nlh_context_state_seed_self_ref(mems.data_ptr(), get("m_k_init"), get("m_v_init"), get("m_q_init"),
                                                    get("m_eta_init"), get("m_alpha_init"), get("m_mem_init"), chains, d)
            elif mems is not None and mm is not None:
                chains, six, d, _ = mems.shape
                lib.nlh_context_state_seed_self_ref(mems.data_ptr(), None, None, None, None, None, mm.data_ptr(), chains, d)
            if mm is not None and lv < len(self.memory) and self.memory[lv] is not None:
                mem = self.memory[lv]
                if mem.numel() % mm.numel() == 0 and mem.numel() >= mm.numel():
                    mem.view(-1, mm.numel()).copy_(mm.reshape(1, -1).expand(mem.numel() // mm.numel(), -1))

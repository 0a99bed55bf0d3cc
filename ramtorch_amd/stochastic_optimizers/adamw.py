"""``ramtorch.AdamW`` on MI355X: the same optimizer interface as the reference's
``ramtorch/stochastic_optimizers/adamw.py`` (constructor arguments, ``param_groups``,
``state[p] = {"step", "ema", "ema_squared"}``, ``step()``, inherited
``state_dict`` / ``load_state_dict``), with the per-tensor loop of torch ops
replaced by one fused HIP launch over all tensors (GPU-resident tensors) or by
a chunked H2D / update / D2H pipeline (tensors held in host memory).

There is no CPU or eager fallback: ``step()`` needs the HIP library and a GPU.
"""
from __future__ import annotations

import time
from typing import Dict, List, Optional

import numpy as np
import torch
from torch.optim import Optimizer

from .. import _gather as G
from .. import _native as N
from .. import functional as F

_handles: Dict[int, N.Handle] = {}


def _handle(device_index: int) -> N.Handle:
    h = _handles.get(device_index)
    if h is None:
        h = _handles[device_index] = N.Handle(device_index)
    return h


class _Rec:
    """Static facts about one parameter and its two states (see AdamW._make_rec)."""
    __slots__ = ("p", "state", "m", "v", "p_ptr", "m_ptr", "v_ptr", "numel", "tensor_id", "dev", "plain", "codes")


def _compute_device_index(p: torch.Tensor) -> int:
    # adamw.py:152-157: CPU params are computed on the current GPU
    if p.is_cuda:
        return p.device.index if p.device.index is not None else torch.cuda.current_device()
    return torch.cuda.current_device()


def copy_stochastic_(target: torch.Tensor, source: torch.Tensor, seed=0, *, noise: Optional[torch.Tensor] = None,
                     reference_noise: bool = False):
    """Stochastically round fp32 ``source`` into bf16 ``target`` (adamw.py:6-30):
    add 16 random bits below the bf16 mantissa, keep the high half.

    The reference draws the bits with ``torch.randint`` from a generator seeded
    with ``seed``; here they come from Philox4x32-10 keyed by ``seed`` (or from
    ``noise``, an int16 tensor, for reproducible tests).  With ``reference_noise`` the
    bits are drawn exactly as the reference draws them (adamw.py:10-21), which makes the
    result bit-identical to the reference's under the same torch build.  The rounding runs on the
    GPU: a CPU ``source`` is uploaded to the current GPU first (the reference rounds wherever
    ``source`` lives, adamw.py:10; here the integer arithmetic is the same and only the place differs),
    a CPU or non-contiguous ``target`` is filled through a GPU temporary.
    """
    if source.dtype != torch.float32 or target.dtype != torch.bfloat16:
        raise TypeError("copy_stochastic_ rounds float32 -> bfloat16")
    if source.numel() != target.numel():
        raise ValueError("target and source sizes differ")
    with torch.no_grad():
        N.lib()
        if not torch.cuda.is_available():
            raise RuntimeError("copy_stochastic_ needs a GPU: the rounding runs only as a HIP kernel")
        if not source.is_cuda:
            # the GPU of the target if it has one, else the current one
            source = source.to(target.device if target.is_cuda else f"cuda:{torch.cuda.current_device()}")
        src = source.contiguous()
        dst = target if (target.is_cuda and target.is_contiguous()) else torch.empty(
            target.shape, dtype=torch.bfloat16, device=source.device)
        nz = None
        if noise is None and reference_noise:
            gen = torch.Generator(device=source.device)
            gen.manual_seed(int(seed))
            noise = torch.randint(low=0, high=(1 << 16), size=source.shape, dtype=torch.int32, device=source.device,
                                  generator=gen).to(torch.int16)  # keeps the low 16 bits
        if noise is not None:
            if noise.dtype not in (torch.int16, torch.uint16) or noise.numel() != source.numel():
                raise ValueError("noise must be an int16 tensor of source's size")
            nz = noise.to(source.device).contiguous()
        with torch.cuda.device(source.device):
            stream = torch.cuda.current_stream().cuda_stream
            N.sr_copy(dst.data_ptr(), src.data_ptr(), src.numel(), None if nz is None else nz.data_ptr(),
                      int(seed) & (2 ** 64 - 1), stream)
        if dst is not target:
            target.copy_(dst)  # bf16 -> bf16, exact
    return target


class AdamW(Optimizer):
    r"""AdamW with bf16 stochastic rounding of parameters and states.

    Arguments (same meaning and defaults as the reference, adamw.py:57-69):
        params: iterable of parameters or of param-group dicts (for instance one
            rank's list from ``create_zero_param_groups``; empty groups are fine).
        lr (float, default 1e-3), betas (default (0.9, 0.999)), eps (default 1e-8),
        weight_decay (default 1e-2): decoupled decay, applied as
            ``p *= 1 - (lr / bias_correction) * weight_decay`` (adamw.py:188,198).
        centralization (default 0): subtract ``c *`` row mean from each gradient.
        chunk_size (default 64): kept for interface compatibility; the fused step
            has no per-tensor synchronisation to space out.
        dtype (default bfloat16): dtype of ``ema`` / ``ema_squared``.
        storage_device (default "cpu"): where the states live; "cpu" states are pinned.

    Keyword-only additions (not in the reference):
        seed: Philox key of the rounding noise.
        stream_chunk_bytes: bytes of bf16 per staged chunk of the host-resident path.
        loss_scale: gradients are divided by this inside the kernel.
        max_grad_norm: global L2 clip computed on the GPU before the update.  A non-finite norm
            cancels the step on the GPU (nothing is written) and the step counts it had advanced are
            taken back when the next ``step()`` begins (``step_was_skipped()`` tells).
        host_arrays_ordered (attribute, default False): set it when work queued on the current
            stream may still be writing *pinned* host parameters or states when an update is handed
            over with ``step_param`` (a ``p.data.copy_(gpu_tensor, non_blocking=True)``, a weight
            sync): the uploads of such tensors then wait for the stream.  ``step()`` itself always
            waits for the current stream before it uploads anything from host memory.
        noise_source: "philox" (default) draws the rounding noise inside the kernel;
            "reference" draws it the way the reference does -- three ``torch.randint``
            tensors per parameter from generators seeded ``step + 42 / 69 / 420``
            (adamw.py:10-21, 206-218) -- and feeds it to the kernel as explicit noise, so
            that a run is bit-identical to ``ramtorch.AdamW`` under the same torch build
            (with ``centralization`` the row means are then taken with torch's own ``mean``,
            as the reference takes them; the default path uses the library's row-mean kernel,
            whose sums agree with torch's to about 2e-6 relative, not bit for bit).
            A verification mode: it costs the three draws and their memory.
        state_placement: "auto" (default) or "plain".  With GPU-resident states of at least
            ``state_pool_min_bytes`` per kind, "auto" carves all ``ema`` tensors out of one
            pool and all ``ema_squared`` tensors out of another and places the two pools in
            different HBM regions, found by measurement at construction (see
            ``ramtorch_amd/placement.py``; the outcome is in ``state_placement_report``): free device
            memory is taken in chunks of 1 GiB through the library (up to half of what is free, at most
            112 GiB beyond the pools, for up to a second), every chunk is probed with the update's
            traffic against the largest parameter's own memory, the pools are mapped from chunks of
            the two kinds and the rest is given back.  The probe writes the parameter back bit for bit
            as it is; nothing else should be writing parameters meanwhile.
            (The driver clears released memory in the background at about 33 GB/s, and until it
            is done device-wide memory traffic runs about 1 % slower: the first seconds of a run.)
            torch's caching allocator never sees the pools (memory held through the library,
            wrapped as tensors, released with their last views).
            "plain" allocates every state tensor on its own, as the reference does.
    """

    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=1e-2, centralization=0,
                 chunk_size=64, dtype=torch.bfloat16, storage_device="cpu", *, seed: int = 0,
                 stream_chunk_bytes: int = 256 << 20, loss_scale: float = 1.0,
                 max_grad_norm: Optional[float] = None, noise_source: str = "philox",
                 state_placement: str = "auto", state_pool_min_bytes: int = 1 << 30,
                 ema_squared_dtype: Optional[torch.dtype] = None, assume_static_layout: bool = False):
        defaults = dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay, centralization=centralization)
        super().__init__(params, defaults)
        self.chunk_size = chunk_size
        self.optim_state_dtype = dtype
        # the reference keeps both states in one dtype; a wider second moment (bf16 ema, fp32
        # ema_squared) is a common mixed layout and costs nothing extra in the kernel
        self.ema_squared_dtype = dtype if ema_squared_dtype is None else ema_squared_dtype
        self.optim_state_device = storage_device
        self.seed = int(seed)
        self.stream_chunk_bytes = int(stream_chunk_bytes)
        self.loss_scale = float(loss_scale)
        self.max_grad_norm = max_grad_norm
        if noise_source not in ("philox", "reference"):
            raise ValueError(f"noise_source must be 'philox' or 'reference', got {noise_source!r}")
        self.noise_source = noise_source
        self.last_grad_norm: Optional[torch.Tensor] = None  # [norm, clip_coef, found_inf bits, -] on the GPU
        self._skip_check = None           # per device of the last step with max_grad_norm: (event, host copy of the
                                          # norm record, [(state, step count before)]) -- see _settle_skipped_step
        self.last_step_skipped = False    # as of the last _settle_skipped_step()
        self.fuse_in_backward = True      # the hook of make_post_accumulate_hook() is live
        self.host_arrays_ordered = False  # step_param: uploads from pinned host p / m / v wait for the current stream
        self.fuse_row_means = True        # centralization: matrices whose rows fit a wavefront are summed inside the update
        self.max_inflight_bytes = 2 << 30  # gradients kept alive for updates still in flight (step_param)
        self.max_inflight_calls = 2       # staging chunks handed to the copy pipeline and not finished yet
        self._poll_seconds = 0.0002       # completion is read from host memory; no runtime call while waiting
        self.gather_min_tensors = 256     # from this many parameters on, step() gathers descriptors in C++
        self._gather_bufs = {}            # device -> descriptor rows the gatherer fills
        self._gather_stat = None
        self._state_lists = {}
        self._stepped_early = set()       # id(param) updated by step_param since the last step()
        self._inflight = []               # (device, ticket, bytes, tensors kept alive)
        self._early_batch = {}            # device -> [[entry, scalars, handed-over elements], ...], pending elements
        self.assume_static_layout = bool(assume_static_layout)
        self._freeze_requested = self.assume_static_layout
        self._frozen = None               # the recorded layout (see freeze_layout)
        self.layout_refreezes = 0         # how often a frozen layout turned out to have changed
        if state_placement not in ("auto", "plain"):
            raise ValueError(f"state_placement must be 'auto' or 'plain', got {state_placement!r}")
        self.state_placement = state_placement
        self.state_pool_min_bytes = int(state_pool_min_bytes)
        self.state_placement_report = None
        self._state_pools = {}            # "ema" / "ema_squared" -> byte pool; "slots": per parameter, in
                                          # param_groups order: (offset in elements, numel) or None
        # eager state allocation, as adamw.py:84-104
        self._allocate_pooled_states()
        for group in self.param_groups:
            for p in group["params"]:
                if not self.state[p]:
                    self._init_state(p)

    # torch's Optimizer pickles only defaults / state / param_groups; everything this class adds
    # to configure itself travels in one extra entry, so that copies and unpickled optimizers step.
    _CONFIG_DEFAULTS = dict(chunk_size=64, optim_state_dtype=torch.bfloat16, ema_squared_dtype=None,
                            optim_state_device="cpu", seed=0, stream_chunk_bytes=256 << 20, loss_scale=1.0,
                            max_grad_norm=None, noise_source="philox", fuse_in_backward=True, host_arrays_ordered=False,
                            fuse_row_means=True,
                            max_inflight_bytes=2 << 30, max_inflight_calls=2, _poll_seconds=0.0002,
                            gather_min_tensors=256, state_placement="auto", state_pool_min_bytes=1 << 30,
                            assume_static_layout=False)

    def __getstate__(self):
        self._settle_skipped_step()
        self._materialize_frozen_steps()
        st = dict(super().__getstate__())
        st["ramtorch_amd_config"] = {k: getattr(self, k, d) for k, d in self._CONFIG_DEFAULTS.items()}
        return st

    def __setstate__(self, state):
        # Called when unpickling and by load_state_dict (which replaces self.state wholesale):
        # drop everything derived from the state, keep or restore the configuration.
        state = dict(state)
        config = state.pop("ramtorch_amd_config", None)
        super().__setstate__(state)
        if config:
            self.__dict__.update(config)
        for k, d in self._CONFIG_DEFAULTS.items():
            self.__dict__.setdefault(k, d)
        if self.__dict__.get("ema_squared_dtype") is None:
            self.ema_squared_dtype = self.optim_state_dtype
        self._recs = None
        self._desc_cache = {}
        self._state_lists = {}
        self._frozen = None   # steps were materialised by whoever produced `state` (__getstate__ / state_dict)
        self._freeze_requested = bool(self.__dict__.get("assume_static_layout", False))
        self._skip_check = None
        for k, d in (("_state_pools", {}), ("state_placement_report", None), ("_gather_bufs", {}),
                     ("_gather_stat", None), ("last_grad_norm", None), ("layout_refreezes", 0),
                     ("last_step_skipped", False)):
            self.__dict__.setdefault(k, d)
        for k, make in (("_stepped_early", set), ("_inflight", list), ("_early_batch", dict)):
            if k not in self.__dict__:
                self.__dict__[k] = make()

    def state_dict(self):
        """Same layout as the reference (``state`` with ``step / ema / ema_squared`` per
        parameter index, ``param_groups``) plus one extra top-level entry with the Philox
        seed, so that a resumed run draws the noise it would have drawn.  torch's loader
        ignores entries it does not know, so the reference can read these checkpoints."""
        self._settle_skipped_step()
        self._materialize_frozen_steps()
        sd = super().state_dict()
        sd["ramtorch_amd"] = {"seed": self.seed}
        return sd

    def load_state_dict(self, state_dict):
        """torch's loader casts ``ema`` / ``ema_squared`` to the parameter's dtype and
        device and drops pinning, which would silently undo ``dtype=`` /
        ``storage_device=``.  After it has restored steps and hyper-parameters, the two
        states are taken again from the checkpoint itself: original dtype, placed on
        ``storage_device`` (pinned when that is the CPU)."""
        self.unfreeze_layout()
        super().load_state_dict(state_dict)
        extra = state_dict.get("ramtorch_amd")
        if isinstance(extra, dict) and "seed" in extra:
            self.seed = int(extra["seed"])
        saved_ids = [i for g in state_dict["param_groups"] for i in g["params"]]
        ours = [p for g in self.param_groups for p in g["params"]]
        for k_flat, (idx, p) in enumerate(zip(saved_ids, ours)):
            saved = state_dict["state"].get(idx)
            if saved is None:
                continue
            st = self.state[p]
            for k in ("ema", "ema_squared"):
                if k in saved and torch.is_tensor(saved[k]):
                    slot = self._pool_view(k_flat, p, k)
                    if slot is not None and slot.dtype == saved[k].dtype and slot.shape == saved[k].shape:
                        slot.copy_(saved[k])   # keeps the placement chosen at construction
                        st[k] = slot
                        continue
                    t = saved[k].detach().to(device=self.optim_state_device).clone(
                        memory_format=torch.contiguous_format)
                    if self.optim_state_device == "cpu" and torch.cuda.is_available():
                        t = t.pin_memory()
                    st[k] = t
        self._recs = None
        self._desc_cache = {}
        self._state_lists = {}

    # -- a step that the skip flag cancelled must not have counted -------------------------------------
    def _settle_skipped_step(self) -> bool:
        """With ``max_grad_norm``, a non-finite global gradient norm makes the kernels leave everything
        untouched (the GPU decides; the host does not wait for it).  ``state["step"]`` has been advanced
        by then, as adamw.py:177 advances it before the arithmetic -- but a step that did not happen
        must not count: bias corrections and the Philox counter would run one ahead of the data for
        the rest of training (torch's GradScaler never calls ``step()`` on such gradients).  So the
        norm record of a step is copied to pinned host memory behind its kernels, and the next
        ``step()`` (or ``state_dict()``, pickling, ``step_was_skipped()``) reads it -- it landed
        long ago, nothing stalls -- and takes the increments back if the step was cancelled.
        Returns whether it was."""
        checks = self.__dict__.get("_skip_check")
        if not checks:
            return False
        self._skip_check = None
        skipped = False
        for event, host, journal in checks:
            event.synchronize()
            if int(host.view(torch.int32)[2]) != 0:
                skipped = True
                for state, old in reversed(journal):
                    state["step"] = old
        self.last_step_skipped = skipped
        return skipped

    def step_was_skipped(self) -> bool:
        """Whether the most recent ``step()`` was cancelled by a non-finite gradient norm (waits for
        that step's norm pass if it has not finished yet)."""
        if self.__dict__.get("_skip_check"):
            self._settle_skipped_step()
        return self.last_step_skipped

    # -- state ---------------------------------------------------------------------
    def _state_dtype(self, key: str) -> torch.dtype:
        if key == "ema_squared":
            return self.__dict__.get("ema_squared_dtype") or self.optim_state_dtype
        return self.optim_state_dtype

    def _new_state_tensor(self, p: torch.Tensor, key: str = "ema") -> torch.Tensor:
        t = torch.zeros_like(p.data, dtype=self._state_dtype(key), device=self.optim_state_device,
                             memory_format=torch.contiguous_format)
        if self.optim_state_device == "cpu" and torch.cuda.is_available():
            # adamw.py:91-97 pins unconditionally; without a GPU there is nothing to pin for
            t = t.pin_memory()
        return t

    def _allocate_pooled_states(self) -> None:
        """GPU-resident states as views into two pools placed in different HBM regions
        (``state_placement="auto"``).  Leaves ``self.state`` untouched when that does not
        apply; ``_init_state`` then allocates tensor by tensor."""
        if self.state_placement != "auto" or not torch.cuda.is_available():
            return
        try:
            dev = torch.device(self.optim_state_device)
        except (TypeError, RuntimeError):
            return
        if dev.type != "cuda":
            return
        if dev.index is None:
            dev = torch.device("cuda", torch.cuda.current_device())
        params = [p for g in self.param_groups for p in g["params"]]
        esize = {k: torch.empty((), dtype=self._state_dtype(k)).element_size() for k in ("ema", "ema_squared")}
        slots, total = [], 0      # slot offsets in elements (multiples of 256), the same in both pools
        for p in params:
            if self.state[p]:
                slots.append(None)
                continue
            slots.append((total, p.numel()))
            total += (p.numel() + 255) // 256 * 256
        if total * min(esize.values()) < self.state_pool_min_bytes:
            return
        from .. import placement
        N.lib()
        with torch.cuda.device(dev):
            pool_m, pool_v, report = placement.place_pair(_handle(dev.index), dev, total * esize["ema"],
                                                          total * esize["ema_squared"],
                                                          ref=placement.reference_arrays(params, dev))
        self.state_placement_report = report
        self._state_pools = {"ema": pool_m, "ema_squared": pool_v, "slots": slots}
        for k, p in enumerate(params):
            if slots[k] is None:
                continue
            st = self.state[p]
            st["step"] = 0
            st["ema"] = self._pool_view(k, p, "ema")
            st["ema_squared"] = self._pool_view(k, p, "ema_squared")

    def _pool_view(self, k: int, p: torch.Tensor, key: str) -> Optional[torch.Tensor]:
        """The slot of the k-th parameter (param_groups order) in the pool of ``key`` as a
        tensor of p's shape, or None when there is no such slot."""
        pools = self.__dict__.get("_state_pools") or {}
        slots = pools.get("slots") or []
        if key not in pools or k >= len(slots) or slots[k] is None or slots[k][1] != p.numel():
            return None
        off, numel = slots[k]
        es = torch.empty((), dtype=self._state_dtype(key)).element_size()
        return pools[key][off * es:(off + numel) * es].view(self._state_dtype(key)).view(p.shape)

    def _init_state(self, p: torch.Tensor) -> None:
        state = self.state[p]
        state["step"] = 0
        state["ema"] = self._new_state_tensor(p)
        state["ema_squared"] = self._new_state_tensor(p, "ema_squared")

    def _tensor_ids(self) -> Dict[int, int]:
        ids: Dict[int, int] = {}
        k = 0
        for group in self.param_groups:
            for p in group["params"]:
                ids[id(p)] = k
                k += 1
        return ids

    # -- per-parameter records -----------------------------------------------------------
    # What the step needs to know about a parameter and its states does not change from
    # step to step (addresses, sizes, dtypes), so it is gathered once and re-validated
    # cheaply: the state tensors must be the same objects and the parameter's address the same.
    def _make_rec(self, p: torch.Tensor, tensor_id: int) -> "_Rec":
        state = self.state[p]
        if not state:
            self._init_state(p)  # adamw.py:125-148
        m, v = state["ema"], state["ema_squared"]
        r = _Rec()
        r.p, r.state, r.m, r.v, r.tensor_id = p, state, m, v, tensor_id
        r.p_ptr, r.m_ptr, r.v_ptr, r.numel = p.data_ptr(), m.data_ptr(), v.data_ptr(), p.numel()
        r.dev = _compute_device_index(p)
        ok_dt = F._DT_CODE_PMV
        r.plain = (p.is_cuda and m.is_cuda and v.is_cuda and m.device == p.device and v.device == p.device
                   and p.is_contiguous() and m.is_contiguous() and v.is_contiguous()
                   and p.dtype in ok_dt and m.dtype in ok_dt and v.dtype in ok_dt
                   and m.numel() == r.numel and v.numel() == r.numel)
        if r.plain:
            r.codes = (F.dtype_code(p.dtype, "param"), F.dtype_code(m.dtype, "state"), F.dtype_code(v.dtype, "state"))
        return r

    def _records(self) -> List[List["_Rec"]]:
        recs = getattr(self, "_recs", None)
        groups = self.param_groups
        if recs is not None and len(recs) == len(groups) and all(
                len(rg) == len(g["params"]) for rg, g in zip(recs, groups)):
            return recs
        k = 0
        recs = []
        self._positions = {}
        for gi, g in enumerate(groups):
            row = []
            for j, p in enumerate(g["params"]):
                row.append(self._make_rec(p, k))
                self._positions[id(p)] = (gi, j)
                k += 1
            recs.append(row)
        self._recs = recs
        self._desc_cache = {}
        self._state_lists = {}
        return recs

    # -- step ----------------------------------------------------------------------
    def step(self, closure=None, *, noise=None, debug_out=None, grads=None):
        """One optimizer step (adamw.py:106-234).

        ``grads``: optional ``{param: gradient}`` used instead of ``param.grad`` --
        for gradients torch will not store in ``.grad`` (an fp32 gradient of a
        bf16 param, a GPU gradient of a host-resident param).

        ``noise``: optional ``{param: (noise_p, noise_m, noise_v)}`` of int16 GPU
        tensors -- the explicit-noise test mode (every stepped bf16 array needs one).
        ``debug_out``: optional ``{param: (p32, m32, v32)}`` fp32 GPU tensors that
        receive the values before rounding.

        An error raised before the first launch (a sparse or unsupported gradient,
        tensors on different GPUs, an option combination that is not implemented)
        leaves every ``state["step"]`` and every tensor as it was.
        """
        loss = None
        if closure is not None:
            loss = closure()

        N.lib()  # fail loudly before touching any state if the extension is missing
        if not torch.cuda.is_available():
            raise RuntimeError("ramtorch_amd.AdamW.step needs a GPU: the update runs only as HIP kernels")

        self._settle_skipped_step()
        if (self._frozen is not None and noise is None and debug_out is None and grads is None
                and not self._stepped_early and not self._early_batch and not self._inflight):
            if self._step_frozen():
                return loss
        self._materialize_frozen_steps()
        recs = self._records()
        self.finish_early_steps()  # updates started from the backward hook must have landed
        if noise is None and getattr(self, "noise_source", "philox") == "reference":
            noise = self._reference_noise(grads, self._stepped_early)
        # Every step count this call advances is noted, so that they can be put back:
        # (state, old value) from the Python loop, (states, status bytes) from the C++ gatherer.
        journal: list = []
        launched = [False]
        try:
            with torch.no_grad():
                self._step_impl(recs, noise, debug_out, grads, journal, launched)
        except BaseException:
            if not launched[0]:
                for entry in reversed(journal):
                    if len(entry) == 2:
                        entry[0]["step"] = entry[1]
                    else:
                        states, status, written = entry
                        for k in np.flatnonzero(status == written):
                            states[int(k)]["step"] -= 1
            raise
        self._stepped_early.clear()
        return loss

    def _step_impl(self, recs, noise, debug_out, grads, journal, launched) -> None:
        early = self._stepped_early
        scalars: List[N.RtScalars] = []
        scalar_key: Dict[tuple, int] = {}
        # plain lane: tensors wholly on one GPU, contiguous, nothing special -> columns only
        plain: Dict[int, tuple] = {}      # dev -> (recs, grads, grad ptrs, grad codes, steps, scalar idx)
        # general lane: everything else goes through Entry objects
        resident: Dict[int, List[F.Entry]] = {}
        streamed: Dict[int, List[F.Entry]] = {}
        writeback = []  # (destination, contiguous temporary) pairs for non-contiguous p / states
        inv_loss_scale = 1.0 / self.loss_scale if self.loss_scale != 1.0 else 1.0
        extras = noise is not None or debug_out is not None
        dt_code = F._DT_CODE

        # Large groups of plain GPU tensors are walked in C++ when the helper is built; it writes
        # their descriptor rows and advances their step counts, and leaves the rest to the loop below.
        gather = None
        if (grads is None and not extras and not early and self.max_grad_norm is None
                and sum(len(g["params"]) for g in self.param_groups) >= self.gather_min_tensors):
            gather = G.module()
        gathered: Dict[int, list] = {}    # dev -> [descriptor buffer, rows used]
        cen_jobs: Dict[int, list] = {}    # dev -> [(entry, rows, row_len)] of gradients to centralize
        counted: Dict[int, list] = {}     # dev -> [(state, step count before)] of the tensors under max_grad_norm
        skip_checks = []

        for gi, group in enumerate(self.param_groups):
            beta1, beta2 = group["betas"]
            lr, eps, wd, cen = group["lr"], group["eps"], group["weight_decay"], group["centralization"]
            row = recs[gi]
            last_step, last_si = None, -1
            plist = group["params"]
            work = enumerate(plist)
            if gather is not None and cen == 0 and row and row[0].plain and isinstance(plist, list):
                dev = row[0].dev
                slot = gathered.get(dev)
                if slot is None:
                    slot = gathered[dev] = [self._gather_buffer(dev), 0]
                buf, used = slot
                status = self._gather_status(len(plist))
                status[:len(plist)] = gather.PYTHON  # nothing written yet, should the call itself fail
                states = self._state_list(gi)
                journal.append((states, status[:len(plist)], gather.WRITTEN))
                n_rows, new_steps = gather.gather_group(
                    plist, states, dev, buf.ctypes.data + used * buf.itemsize, len(buf) - used,
                    status.ctypes.data, len(scalars), row[0].tensor_id)
                journal[-1] = (states, status[:len(plist)].copy(), gather.WRITTEN)
                slot[1] = used + n_rows
                for st in new_steps:
                    scalar_key[(gi, st, lr, beta1, beta2, eps, wd, cen)] = len(scalars)
                    scalars.append(F.make_scalars(lr, (beta1, beta2), eps, wd, st, centralization=cen,
                                                  inv_loss_scale=inv_loss_scale))
                rest = np.flatnonzero(status[:len(plist)] == gather.PYTHON)
                work = ((int(k), plist[int(k)]) for k in rest)
            for k, p in work:
                grad = grads.get(p, p.grad) if grads is not None else p.grad
                if grad is None:
                    continue  # adamw.py:114: skipped, and its step count does not advance
                if early and id(p) in early:
                    continue  # already updated by step_param() during this backward
                if grad.is_sparse:
                    raise RuntimeError("AdamW does not support sparse gradients")  # adamw.py:118-119
                r = row[k]
                state = r.state
                if (r.p is not p or state.get("ema") is not r.m or state.get("ema_squared") is not r.v
                        or p.data_ptr() != r.p_ptr or r.m.data_ptr() != r.m_ptr or r.v.data_ptr() != r.v_ptr):
                    r = row[k] = self._make_rec(p, r.tensor_id)
                    state = r.state
                step = state["step"] + 1  # adamw.py:177
                journal.append((state, state["step"]))
                if self.max_grad_norm is not None:
                    counted.setdefault(r.dev, []).append(journal[-1])
                state["step"] = step
                if step != last_step:
                    key = (gi, step, lr, beta1, beta2, eps, wd, cen)
                    si = scalar_key.get(key)
                    if si is None:
                        si = scalar_key[key] = len(scalars)
                        scalars.append(F.make_scalars(lr, (beta1, beta2), eps, wd, step, centralization=cen,
                                                      inv_loss_scale=inv_loss_scale))
                    last_step, last_si = step, si
                si = last_si
                dev = r.dev

                gcode = dt_code.get(grad.dtype)
                if (r.plain and cen == 0 and gcode is not None and grad.is_cuda and grad.is_contiguous()
                        and grad.device.index == dev and grad.numel() == r.numel
                        and not (extras and ((noise is not None and p in noise)
                                             or (debug_out is not None and p in debug_out)))):
                    lane = plain.get(dev)
                    if lane is None:
                        lane = plain[dev] = ([], [], [], [], [], [])
                    lane[0].append(r); lane[1].append(grad); lane[2].append(grad.data_ptr())
                    lane[3].append(gcode); lane[4].append(step); lane[5].append(si)
                    continue

                # ---- general lane ----
                arrays = []
                for t in (p.data, r.m, r.v):
                    if t.is_cuda and t.device.index != dev:
                        raise RuntimeError("param and optimizer states live on different GPUs")
                    F.dtype_code(t.dtype, "param")  # an unsupported dtype must raise before anything is launched
                    if not t.is_contiguous():
                        c = t.contiguous()
                        writeback.append((t, c))
                        t = c
                    arrays.append(t)
                g = grad.detach()
                if g.is_cuda and g.device.index != dev:
                    g = g.to(f"cuda:{dev}")
                if not g.is_contiguous():
                    g = g.contiguous()
                if g.dtype not in (torch.bfloat16, torch.float32, torch.float16):
                    g = g.to(torch.float32)  # adamw.py:167 upcasts every gradient to fp32
                if self.max_grad_norm is not None and not g.is_cuda:
                    # the global norm is taken on the GPU: a host gradient is shipped once, here, and
                    # the update then reads the device copy
                    g = g.to(f"cuda:{dev}", non_blocking=True)
                e = F.Entry(p=arrays[0], g=g, m=arrays[1], v=arrays[2], step=step, scalars_idx=si,
                            tensor_id=r.tensor_id)
                if cen != 0:
                    if not g.is_cuda:
                        g = g.to(f"cuda:{dev}", non_blocking=True)
                        e.g = g
                    if getattr(self, "noise_source", "philox") == "reference" and inv_loss_scale == 1.0:
                        e.row_mean, e.row_len = self._row_means(g, dev, inv_loss_scale)   # torch's own mean
                    elif g.numel():
                        # adamw.py:179-184: mean over every dim but the first (over all of them for 0-d / 1-d)
                        rows = g.shape[0] if g.dim() >= 2 else 1
                        row_len = g.numel() // rows if rows else 0
                        if noise is not None and p in noise:
                            e.noise = tuple(noise[p])
                        if debug_out is not None and p in debug_out:
                            e.dbg = tuple(debug_out[p])
                        if (self.__dict__.get("fuse_row_means", True) and e.p.is_cuda and e.m.is_cuda and e.v.is_cuda
                                and F.rowwise_ok(e, row_len, explicit_noise=noise is not None)):
                            e.row_len = row_len     # the update kernel sums the rows itself: no separate pass
                        else:
                            # the rows of all such gradients of the step are summed in one launch below
                            cen_jobs.setdefault(dev, []).append((e, rows, row_len))
                if noise is not None and p in noise:
                    e.noise = tuple(noise[p])
                if debug_out is not None and p in debug_out:
                    e.dbg = tuple(debug_out[p])
                on_gpu = e.p.is_cuda and e.g.is_cuda and e.m.is_cuda and e.v.is_cuda
                (resident if on_gpu else streamed).setdefault(dev, []).append(e)

        for dev, jobs in cen_jobs.items():
            with torch.cuda.device(dev):
                F.row_means_multi(_handle(dev), jobs, inv_loss_scale)   # writes fresh buffers only

        # ---- everything that can still raise for a bad argument happens before the first launch
        explicit = noise is not None
        work_by_dev = []
        for dev in sorted(set(plain) | set(resident) | set(streamed) | set(gathered)):
            res, stm = resident.get(dev, []), streamed.get(dev, [])
            lane = plain.get(dev)
            descs = self._plain_descs(dev, lane) if lane is not None else None
            if dev in gathered and gathered[dev][1]:
                d0 = gathered[dev][0][:gathered[dev][1]]
                descs = d0 if descs is None else np.concatenate([d0, descs])
            if res:
                d2 = F.pack_descs(res, streamed=False)
                descs = d2 if descs is None else np.concatenate([descs, d2])
            stm_descs = F.pack_descs(stm, streamed=True) if stm else None
            work_by_dev.append((dev, lane, res, stm, descs, stm_descs))

        for dev, lane, res, stm, descs, stm_descs in work_by_dev:
            h = _handle(dev)
            with torch.cuda.device(dev):
                clip = skip = None
                if self.max_grad_norm is not None:
                    # one norm over every gradient of the step, wherever its parameter lives
                    gl = (lane[1] if lane is not None else []) + [e.g for e in res] + [e.g for e in stm]
                    out = F.grad_norm(h, gl, inv_loss_scale=inv_loss_scale, max_norm=self.max_grad_norm)
                    self.last_grad_norm = out
                    clip, skip = out[1:2], out[2:3]
                    # the record goes to pinned host memory behind the norm pass; the next step reads it there
                    host = torch.empty(4, dtype=torch.float32, pin_memory=True)
                    host.copy_(out, non_blocking=True)
                    event = torch.cuda.Event()
                    event.record()
                    skip_checks.append((event, host, counted.get(dev, [])))
                launched[0] = True
                if descs is not None:
                    F.launch_resident(h, descs, scalars, seed=self.seed, explicit_noise=explicit, clip_coef=clip,
                                      skip=skip)
                if stm:
                    chunk_elems = max(8, (self.stream_chunk_bytes // 2) // 8 * 8)
                    F.step_streamed(h, stm, scalars, seed=self.seed, explicit_noise=explicit,
                                    chunk_elems=chunk_elems, clip_coef=clip, skip=skip, descs=stm_descs)
        for dst, tmp in writeback:
            dst.copy_(tmp)
        if skip_checks:
            self._skip_check = skip_checks
        if self._freeze_requested:
            self._record_layout(gathered, plain, resident, streamed, scalar_key, explicit)

    # -- a recorded layout: steps that only check that nothing moved ----------------------------------
    def freeze_layout(self) -> None:
        """Record, at the next ``step()``, which tensors stepped and where they lie, and from then on
        only *check* that per step instead of gathering it again: every parameter and gradient must
        still be at its recorded address (a C++ walk of about 50 ns per tensor instead of 230 ns),
        hyper-parameters are re-read per group as always, step counts advance in bulk.  For parameter
        sets of thousands of small tensors whose gradients keep their storage from step to step
        (``zero_grad(set_to_none=False)`` or gradients accumulated in place).

        Applies to steps that the C++ gatherer covers completely: one GPU, at least
        ``gather_min_tensors`` parameters, every stepping tensor plain (contiguous, on the GPU), no
        ``centralization`` / ``max_grad_norm`` / ``noise_source="reference"`` / ``step_param``.
        Otherwise nothing is recorded and steps run as usual.

        What ends a recorded layout: ``add_param_group``, ``load_state_dict``, ``unfreeze_layout()``,
        and any step whose check fails (a gradient appeared, vanished, moved or changed dtype; a
        parameter moved; a ``params`` list changed; an entry of ``optimizer.state`` or of a
        parameter's state dict was assigned, added or removed) -- that step runs the full path, with
        the same results, and records the layout again if ``assume_static_layout`` is set.  Not
        seen: the storage of a state tensor exchanged in place (``state["ema"].data = ...``,
        ``set_``); the recorded storages are kept alive, so such a step still updates the memory that
        was recorded.  While a layout is
        recorded, ``state[p]["step"]`` of the recorded tensors lags behind; it is brought up to date
        by ``state_dict()``, ``unfreeze_layout()`` and by any step that takes the full path."""
        self._freeze_requested = True

    def unfreeze_layout(self) -> None:
        self._materialize_frozen_steps()
        self._frozen = None
        self._freeze_requested = bool(self.__dict__.get("assume_static_layout", False))

    def add_param_group(self, param_group):
        if self.__dict__.get("_frozen") is not None:
            self.unfreeze_layout()
        super().add_param_group(param_group)

    def _materialize_frozen_steps(self) -> None:
        fz = self.__dict__.get("_frozen")
        if fz is None or fz["pending"] == 0:
            return
        k = fz["pending"]
        for st in fz["states"]:
            st["step"] += k
        # the recorded step counts move along, so that the next recorded step builds its scalars
        # for the step it really is (the descriptors' own step words have advanced all the while)
        fz["keys"] = [(gi, st + k) for gi, st in fz["keys"]]
        fz["pending"] = 0
        # these writes are the optimizer's own: the state dicts' modification stamps are taken again
        G.module().dict_versions(fz["state_dicts"], fz["versions"].ctypes.data, len(fz["state_dicts"]))

    def _record_layout(self, gathered, plain, resident, streamed, scalar_key, explicit) -> None:
        self._frozen = None
        if (explicit or plain or resident or streamed or len(gathered) != 1 or self.max_grad_norm is not None
                or G.module() is None or not hasattr(G.module(), "verify_layout")):
            return
        (dev, (buf, rows)), = gathered.items()
        if rows == 0:
            return
        descs = buf[:rows].copy()
        params = [p for g in self.param_groups for p in g["params"]]
        first_id = {}
        k = 0
        for gi, g in enumerate(self.param_groups):
            first_id[gi] = k
            k += len(g["params"])
        expect = np.zeros((len(params), 3), np.uint64)
        expect[:, 0] = [p.data_ptr() for p in params]
        ids = descs["tensor_id"].astype(np.int64)
        if len(np.unique(ids)) != rows or ids.max() >= len(params):
            return
        expect[ids, 1] = descs["g"]
        expect[ids, 2] = descs["g_dtype"]
        # every row's p must be the parameter with its tensor_id (the gatherer numbers them in order)
        if not np.array_equal(expect[ids, 0], descs["p"]):
            return
        keys = [None] * len(scalar_key)
        for (gi, st, *_), idx in scalar_key.items():
            keys[idx] = (gi, st)
        if any(x is None for x in keys):
            return
        # The descriptors keep the addresses of the state tensors.  Their storages are held, so that the
        # addresses stay valid whatever happens to the tensors, and every state dict's modification
        # stamp is noted (with that of ``self.state`` itself): a state that is replaced, removed or
        # added shows there, one load per dict and step.
        states = [self.state[params[i]] for i in ids]
        state_dicts = states + [self.state]
        versions = np.zeros(len(state_dicts), np.uint64)
        try:
            G.module().dict_versions(state_dicts, versions.ctypes.data, len(state_dicts))
        except (NotImplementedError, AttributeError):
            return    # no stamps in this interpreter (or an older helper): no recorded layouts
        keep = [t.untyped_storage() for st in states for t in (st["ema"], st["ema_squared"])]
        self._frozen = {"dev": dev, "descs": descs, "params": params, "expect": expect,
                        "states": states, "state_dicts": state_dicts, "versions": versions, "keep": keep,
                        "keys": keys, "pending": 0,
                        "group_lists": [(g["params"], len(g["params"])) for g in self.param_groups]}
        if not self.assume_static_layout:
            self._freeze_requested = False

    def _step_frozen(self) -> bool:
        """One step over the recorded layout; False (and the record dropped) when anything moved."""
        fz = self._frozen
        groups = self.param_groups
        ok = len(groups) == len(fz["group_lists"]) and all(
            g["params"] is lst and len(lst) == n and g["centralization"] == 0
            for g, (lst, n) in zip(groups, fz["group_lists"]))
        ok = ok and self.max_grad_norm is None and getattr(self, "noise_source", "philox") == "philox"
        if ok:
            ok = (fz["state_dicts"][-1] is self.state
                  and G.module().verify_versions(fz["state_dicts"], fz["versions"].ctypes.data, len(fz["state_dicts"]))
                  and G.module().verify_layout(fz["params"], fz["expect"].ctypes.data, len(fz["params"])))
        if not ok:
            self.layout_refreezes += 1
            self.unfreeze_layout()
            self._freeze_requested = self._freeze_requested or self.assume_static_layout
            return False
        ahead = fz["pending"] + 1
        inv_loss_scale = 1.0 / self.loss_scale if self.loss_scale != 1.0 else 1.0
        scalars = []
        for gi, st in fz["keys"]:
            g = groups[gi]
            scalars.append(F.make_scalars(g["lr"], tuple(g["betas"]), g["eps"], g["weight_decay"], st + ahead,
                                          inv_loss_scale=inv_loss_scale))
        descs = fz["descs"]
        descs["step"] += 1    # uint32: wraps like the mask of the full path
        dev = fz["dev"]
        try:
            with torch.no_grad(), torch.cuda.device(dev):
                F.launch_resident(_handle(dev), descs, scalars, seed=self.seed, explicit_noise=False)
        except BaseException:
            descs["step"] -= 1
            raise
        fz["pending"] = ahead
        return True

    def _reference_noise(self, grads, early) -> dict:
        """The reference's own rounding noise for every parameter about to step: a fresh
        generator on the compute device seeded ``step + 42`` (param), ``+ 69`` (ema), ``+ 420``
        (ema_squared) with the step count after the increment, ``randint(0, 65536)`` of the
        parameter's shape (adamw.py:10-21, 177, 206-218).  Returned as int16 bit patterns."""
        out = {}
        for group in self.param_groups:
            for p in group["params"]:
                grad = grads.get(p, p.grad) if grads is not None else p.grad
                if grad is None or (early and id(p) in early):
                    continue
                state = self.state[p]
                if not state:
                    self._init_state(p)
                step = state["step"] + 1
                dev = torch.device("cuda", _compute_device_index(p))
                draws = []
                for is_bf16, offset in ((p.dtype == torch.bfloat16, 42), (state["ema"].dtype == torch.bfloat16, 69),
                                        (state["ema_squared"].dtype == torch.bfloat16, 420)):
                    if not is_bf16:
                        draws.append(None)  # written back with a plain copy_: no noise drawn (adamw.py:208,221)
                        continue
                    gen = torch.Generator(device=dev)
                    gen.manual_seed(step + offset)
                    r = torch.randint(low=0, high=(1 << 16), size=p.shape, dtype=torch.int32, device=dev, generator=gen)
                    draws.append(r.to(torch.int16).view(-1))  # keeps the low 16 bits
                out[p] = tuple(draws)
        return out

    # -- updating one parameter as soon as its gradient exists --------------------------------
    def make_post_accumulate_hook(self):
        """A callable for ramtorch's ``_ramtorch_post_accumulate_grad_hooks``
        (``linear.py:97-111``: called as ``hook(param)`` inside ``Linear.backward`` while
        ``param.ramtorch_grad`` holds the accumulated gradient on the GPU).  It runs the
        update of that parameter right there, from the GPU gradient, instead of waiting
        for ``step()`` to ship the gradient back from the CPU (``adamw.py:167``).  Set
        ``optimizer.fuse_in_backward = False`` during gradient-accumulation micro-steps.
        ``step()`` afterwards waits for these updates and skips the parameters they covered."""
        def hook(param):
            if self.fuse_in_backward:
                grad = getattr(param, "ramtorch_grad", None)
                self.step_param(param, grad if grad is not None else param.grad)
        return hook

    def _row_means(self, g: torch.Tensor, dev: int, inv_loss_scale: float):
        """(fp32 row means of the GPU gradient ``g``, row length) for centralization, adamw.py:179-184:
        the mean over every dim but the first (over all of them for 0-d / 1-d)."""
        rows = g.shape[0] if g.dim() >= 2 else 1
        row_len = g.numel() // rows if rows else 0
        if not g.numel():
            return None, 0
        if getattr(self, "noise_source", "philox") == "reference" and inv_loss_scale == 1.0:
            # the verification mode reproduces the reference bit for bit: the means come
            # from the very call the reference makes (a sum's bits depend on its order)
            g32 = g.to(torch.float32)
            return g32.mean(dim=tuple(range(1, g32.dim())), keepdim=True).reshape(-1).contiguous(), row_len
        with torch.cuda.device(dev):
            return F.row_means(_handle(dev), g, rows, row_len, inv_loss_scale), row_len

    def step_param(self, p: torch.Tensor, grad: Optional[torch.Tensor] = None) -> None:
        """Update one parameter now, without waiting: same arithmetic, same noise and same
        ``state["step"]`` bookkeeping as ``step()`` would apply to it.  The update is queued
        behind the work already on the current stream; host-resident arrays are final after
        ``finish_early_steps()`` (``step()`` calls it)."""
        N.lib()
        if not torch.cuda.is_available():
            raise RuntimeError("ramtorch_amd.AdamW.step_param needs a GPU: the update runs only as HIP kernels")
        if grad is None:
            grad = p.grad
        if grad is None:
            return
        if grad.is_sparse:
            raise RuntimeError("AdamW does not support sparse gradients")
        if self.max_grad_norm is not None:
            raise NotImplementedError("step_param with max_grad_norm (the global norm needs every gradient)")
        if id(p) in self._stepped_early:
            raise RuntimeError("step_param called twice for one parameter without a step() in between")
        if self.__dict__.get("_frozen") is not None:
            # a recorded layout does not cover steps of single parameters, and while it is in use the
            # step counts in the states lag: bring them up to date before one of them is read
            self.unfreeze_layout()
        recs = self._records()
        pos = self._positions.get(id(p))
        if pos is None:
            raise ValueError("step_param: tensor is not a parameter of this optimizer")
        gi, k = pos
        group = self.param_groups[gi]
        r = recs[gi][k]
        state = r.state
        if (state.get("ema") is not r.m or state.get("ema_squared") is not r.v or p.data_ptr() != r.p_ptr
                or r.m.data_ptr() != r.m_ptr or r.v.data_ptr() != r.v_ptr):
            r = recs[gi][k] = self._make_rec(p, r.tensor_id)
            state = r.state
        if not (p.is_contiguous() and r.m.is_contiguous() and r.v.is_contiguous()):
            raise NotImplementedError("step_param needs contiguous parameter and state tensors")
        dev = r.dev
        with torch.no_grad():
            g = grad.detach()
            if not g.is_cuda or g.device.index != dev:
                g = g.to(f"cuda:{dev}", non_blocking=True)
            if not g.is_contiguous():
                g = g.contiguous()
            if g.dtype not in (torch.bfloat16, torch.float32, torch.float16):
                g = g.to(torch.float32)
            old_step = state["step"]
            step = old_step + 1    # adamw.py:177; written to the state only when nothing can raise any more
            inv_loss_scale = 1.0 / self.loss_scale if self.loss_scale != 1.0 else 1.0
            cen = group["centralization"]
            sc = [F.make_scalars(group["lr"], tuple(group["betas"]), group["eps"], group["weight_decay"], step,
                                 centralization=cen, inv_loss_scale=inv_loss_scale)]
            e = F.Entry(p=p.data, g=g, m=r.m, v=r.v, step=step, scalars_idx=0, tensor_id=r.tensor_id,
                        ordered=bool(self.__dict__.get("host_arrays_ordered", False)))
            for t, what in ((e.p, "param"), (e.g, "grad"), (e.m, "state"), (e.v, "state")):
                F.dtype_code(t.dtype, what)     # an unsupported dtype raises here
            if g.numel() != p.numel():
                raise ValueError("step_param: the gradient's size differs from the parameter's")
            if cen != 0 and g.numel():
                rows = g.shape[0] if g.dim() >= 2 else 1
                if (self.__dict__.get("fuse_row_means", True) and e.p.is_cuda and e.m.is_cuda and e.v.is_cuda
                        and getattr(self, "noise_source", "philox") == "philox" and F.rowwise_ok(e, g.numel() // rows)):
                    e.row_len = g.numel() // rows    # the update kernel sums the rows itself
                else:
                    e.row_mean, e.row_len = self._row_means(g, dev, inv_loss_scale)
            h = _handle(dev)
            state["step"] = step
            handed_over = False    # part of this tensor is already on the copy pipeline: the step counts
            try:
                with torch.cuda.device(dev):
                    if e.p.is_cuda and e.m.is_cuda and e.v.is_cuda:
                        F.step_resident(h, [e], sc, seed=self.seed, explicit_noise=False)  # stream-ordered already
                    else:
                        # Tensors are handed to the copy pipeline in pieces of exactly one staging chunk
                        # (a tensor may be cut, at a multiple of 8 elements): chunks of equal size keep
                        # H2D and D2H overlapped, a run of unequal tensors would not.
                        batch = self._early_batch.setdefault(dev, [[], 0])
                        batch[0].append([e, sc[0], 0])      # entry, its scalars, elements already handed over
                        batch[1] += e.p.numel()
                        try:
                            self._flush_early_batch(dev, final=False)
                        except BaseException:
                            # nothing of this tensor has been handed over unless a piece of it was: take it
                            # out of the batch again when it is still whole
                            if batch[0] and batch[0][-1][0] is e and batch[0][-1][2] == 0:
                                batch[0].pop()
                                batch[1] -= e.p.numel()
                                if not batch[0]:
                                    self._early_batch.pop(dev, None)
                            else:
                                handed_over = True
                            raise
            except BaseException:
                if not handed_over:
                    state["step"] = old_step
                raise
        self._stepped_early.add(id(p))

    def _flush_early_batch(self, dev: int, final: bool) -> None:
        batch = self._early_batch.get(dev)
        if not batch:
            return
        chunk_elems = max(8, (self.stream_chunk_bytes // 2) // 8 * 8)
        h = _handle(dev)
        while batch[0] and (batch[1] >= chunk_elems or final):
            room = chunk_elems
            entries, scalars = [], []
            while batch[0] and room >= 8:
                item = batch[0][0]
                e, sc, used = item
                n = e.p.numel()
                take = min(n - used, room)
                if take < n - used:
                    take -= take % 8            # a cut must fall on a Philox block boundary
                    if take == 0:
                        break
                if used == 0 and take == n:
                    piece = e
                else:
                    sl = slice(used, used + take)
                    piece = F.Entry(p=e.p.view(-1)[sl], g=e.g.view(-1)[sl], m=e.m.view(-1)[sl], v=e.v.view(-1)[sl],
                                    step=e.step, scalars_idx=0, tensor_id=e.tensor_id, row_mean=e.row_mean,
                                    row_len=e.row_len, elem_offset=e.elem_offset + used, keep=[e])
                piece.scalars_idx = len(scalars)
                scalars.append(sc)
                entries.append(piece)
                room -= take
                room -= room % 8                # the next piece starts 16-byte aligned in staging
                batch[1] -= take
                if used + take == n:
                    batch[0].pop(0)
                else:
                    item[2] = used + take
            if not entries:
                break
            self._wait_for_room(dev)
            with torch.cuda.device(dev):
                ticket = F.step_streamed(h, entries, scalars, seed=self.seed, explicit_noise=False,
                                         chunk_elems=chunk_elems, wait=False)
            nbytes = sum(x.g.numel() * x.g.element_size() for x in entries)
            self._inflight.append((dev, ticket, nbytes, entries))
        if not batch[0]:
            self._early_batch.pop(dev, None)

    def _wait_for_room(self, dev: int) -> None:
        """Drop the references of finished asynchronous updates and wait until fewer than
        ``max_inflight_calls`` chunks are in flight.  Two chunks keep both staging buffers
        busy (the next H2D overlaps the previous D2H); on the test machine a third chunk
        queued while two are running made individual copies four times slower.  Completion
        is a number the pipeline writes into pinned host memory, so waiting for it never
        enters the runtime."""
        h = _handle(dev)
        last_done, last_change = -1, time.monotonic()
        while True:
            done = h.streamed_completed()
            self._inflight = [x for x in self._inflight if not (x[0] == dev and x[1] <= done)]
            mine = [x for x in self._inflight if x[0] == dev]
            if len(mine) < self.max_inflight_calls and sum(x[2] for x in mine) <= self.max_inflight_bytes:
                return
            if done != last_done:
                last_done, last_change = done, time.monotonic()
            elif time.monotonic() - last_change > 60.0:
                # no chunk has finished for a minute: fall back to a blocking wait, which
                # either returns or raises the device error behind the stall
                with torch.cuda.device(dev):
                    h.streamed_wait()
                last_change = time.monotonic()
            time.sleep(self._poll_seconds)

    def finish_early_steps(self) -> None:
        """Wait until every update started by ``step_param`` has landed in host memory."""
        for dev in list(self._early_batch):
            self._flush_early_batch(dev, final=True)
        for dev in sorted({x[0] for x in self._inflight}):
            with torch.cuda.device(dev):
                _handle(dev).streamed_wait()
        self._inflight = []

    def _gather_buffer(self, dev: int) -> np.ndarray:
        """Descriptor rows the C++ gatherer fills for one device (one row per parameter at most)."""
        n = sum(len(g["params"]) for g in self.param_groups)
        buf = self._gather_bufs.get(dev)
        if buf is None or len(buf) < n:
            buf = self._gather_bufs[dev] = np.zeros(n, F.DESC_DTYPE)
        return buf

    def _gather_status(self, n: int) -> np.ndarray:
        st = self._gather_stat
        if st is None or len(st) < n:
            st = self._gather_stat = np.zeros(n, np.uint8)
        return st

    def _state_list(self, gi: int) -> list:
        """The state dicts of group ``gi`` in parameter order (cached with the records)."""
        lst = self._state_lists.get(gi)
        if lst is None or len(lst) != len(self._recs[gi]):
            lst = self._state_lists[gi] = [r.state for r in self._recs[gi]]
        return lst

    def _plain_descs(self, dev: int, lane) -> np.ndarray:
        """Descriptor array of the plain lane.  The columns that describe p / m / v are
        reused from the previous step when the same records step again."""
        lrecs, _, gptrs, gcodes, steps, sis = lane
        key = tuple(map(id, lrecs))
        cached = self._desc_cache.get(dev)
        if cached is not None and cached[0] == key:
            d = cached[1]
        else:
            d = np.zeros(len(lrecs), F.DESC_DTYPE)
            d["p"] = [r.p_ptr for r in lrecs]
            d["m"] = [r.m_ptr for r in lrecs]
            d["v"] = [r.v_ptr for r in lrecs]
            d["numel"] = [r.numel for r in lrecs]
            d["tensor_id"] = [r.tensor_id for r in lrecs]
            d["p_dtype"] = [r.codes[0] for r in lrecs]
            d["m_dtype"] = [r.codes[1] for r in lrecs]
            d["v_dtype"] = [r.codes[2] for r in lrecs]
            self._desc_cache[dev] = (key, d, lrecs)  # lrecs keeps the ids in `key` alive
        d["g"] = gptrs
        d["g_dtype"] = gcodes
        d["step"] = np.asarray(steps, dtype=np.uint64) & 0xFFFFFFFF
        d["scalars_idx"] = sis
        return d

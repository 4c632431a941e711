"""The optimizer step of the train loop in two kernel passes: gradient-norm clipping + Adam.

Stands where the reference's trainer calls ``torch.nn.utils.clip_grad_norm_(model.parameters(), max_norm=1.0)``
and then ``optimizer.step()`` on ``torch.optim.Adam(..., fused=True)`` (``ScaFFold/utils/trainer.py:678-694``,
``:268-274``).  Same arithmetic (torch's Adam formulas, bias corrections from a step counter that lives on the
device, the clipping factor ``min(1, max_norm / (norm + 1e-6))``), but the gradients are scaled on the fly instead
of being rewritten, the norm is a fixed-order sum (bitwise reproducible), and the whole step is two launches per 64
tensors with nothing that synchronises, so it can be captured in a graph.

``state_dict()`` has the layout of ``torch.optim.Adam`` (``step``, ``exp_avg``, ``exp_avg_sq`` per parameter), so
checkpoints move between the two.
"""

from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import _lib
from ._lib import AdamDesc

__all__ = ["FusedClipAdam"]


def _ptr_array(tensors):
    arr = (ctypes.c_void_p * len(tensors))()
    for i, t in enumerate(tensors):
        arr[i] = None if t is None else t.data_ptr()
    return arr


class FusedClipAdam(torch.optim.Optimizer):
    """``clip_grad_norm_(params, max_norm)`` + ``Adam.step()`` fused. fp32 parameters on one GPU only.

    ``max_norm=None`` disables clipping. ``shadow_dtype`` (``torch.bfloat16`` / ``torch.float16``) keeps a
    half-precision copy of every parameter, refreshed by the update kernel itself, in ``self.shadow[param]``.
    After ``step()``, ``self.grad_norm`` holds the unclipped total gradient norm (a 0-dim device tensor, what
    ``clip_grad_norm_`` returns)."""

    def __init__(self, params, lr: float = 1e-3, betas=(0.9, 0.999), eps: float = 1e-8, weight_decay: float = 0.0,
                 max_norm: Optional[float] = None, shadow_dtype: Optional[torch.dtype] = None):
        if lr < 0.0 or eps < 0.0 or weight_decay < 0.0:
            raise ValueError(f"invalid hyperparameter: lr={lr} eps={eps} weight_decay={weight_decay}")
        if not (0.0 <= betas[0] < 1.0 and 0.0 <= betas[1] < 1.0):
            raise ValueError(f"invalid betas {betas}")
        if max_norm is not None and not max_norm > 0.0:
            raise ValueError(f"max_norm must be positive or None, got {max_norm}")
        if shadow_dtype not in (None, torch.bfloat16, torch.float16):
            raise ValueError(f"shadow_dtype must be bfloat16, float16 or None, got {shadow_dtype}")
        super().__init__(params, dict(lr=lr, betas=tuple(betas), eps=eps, weight_decay=weight_decay))
        self.max_norm = max_norm
        self.shadow_dtype = shadow_dtype
        self.shadow = {}
        if shadow_dtype is not None:
            self.refresh_shadows()
        self.grad_norm = None
        self._slots = None
        self._plans = {}
        self._pack_plan = None

    @torch.no_grad()
    def refresh_shadows(self):
        """(Re)makes the half-precision copy of every parameter and publishes it on the parameter, where
        ``FastConv3d`` / ``FastConvTranspose3d`` find it under autocast. Needed only after the parameters were
        changed behind torch's back (``.data`` writes); ordinary in-place updates are noticed through the version
        counter and simply fall back to the per-call cast until the next ``step()``."""
        if self.shadow_dtype is None:
            return
        for group in self.param_groups:
            for p in group["params"]:
                if p.dtype is not torch.float32 or not p.is_cuda:
                    continue
                sh = self.shadow.get(p)
                if sh is None:
                    sh = self.shadow[p] = torch.empty_like(p, dtype=self.shadow_dtype, memory_format=torch.preserve_format)
                sh.copy_(p)
                p._sfh_shadow = sh
                p._sfh_shadow_version = p._version

    @staticmethod
    def _dense(t):
        return t.is_contiguous() or (t.dim() == 5 and t.is_contiguous(memory_format=torch.channels_last_3d))

    def _check(self, p):
        if not p.is_cuda or p.dtype is not torch.float32 or not self._dense(p):
            raise NotImplementedError(f"FusedClipAdam: parameter must be a dense fp32 GPU tensor, got {p.dtype} on {p.device} "
                                      f"with strides {tuple(p.stride())}")

    def _state_of(self, p):
        st = self.state[p]
        if not st:
            # One counter tensor for all parameters whose state is created before the first step (torch keeps one per
            # parameter, all equal; state_dict() shows the same values either way): the kernels advance it once, and
            # no multi-tensor add is needed for the others.
            fresh = self.__dict__.get("_fresh_step")
            if fresh is None or fresh[0].device != p.device or fresh[1]:
                fresh = self._fresh_step = [torch.zeros((), dtype=torch.float32, device=p.device), False]
            st["step"] = fresh[0]
            st["exp_avg"] = torch.zeros_like(p, memory_format=torch.preserve_format)
            st["exp_avg_sq"] = torch.zeros_like(p, memory_format=torch.preserve_format)
        self._check_state(p, st)
        return st

    @staticmethod
    def _other_steps(states):
        """The step tensors that are not the first parameter's, each once."""
        seen, out = {id(states[0]["step"])}, []
        for st in states[1:]:
            if id(st["step"]) not in seen:
                seen.add(id(st["step"]))
                out.append(st["step"])
        return out

    def _plan(self, active, device):
        """Pointer tables of everything that does not move between steps (parameters, moments, shadow copies),
        built once per set of active parameters."""
        key = tuple(id(p) for _, p in active)
        plan = self._plans.get(key)
        if plan is not None:
            return plan
        L = _lib.lib()
        params = [p for _, p in active]
        for p in params:
            if p.device != device:
                raise NotImplementedError("FusedClipAdam: all parameters must live on one device")
            self._check(p)
        states = [self._state_of(p) for p in params]
        numel = (ctypes.c_int64 * len(params))(*[p.numel() for p in params])
        plan = {
            "params": params, "states": states, "numel": numel, "nslots": int(L.sfh_adam_slots(len(params), numel)),
            "others": self._other_steps(states), "groups": [],
        }
        for group in self.param_groups:
            idx = [i for i, (g, _) in enumerate(active) if g is group]
            if not idx:
                continue
            gp = [params[i] for i in idx]
            shadows = None
            if self.shadow_dtype is not None:
                for p in gp:
                    if p not in self.shadow:
                        self.shadow[p] = torch.empty_like(p, dtype=self.shadow_dtype, memory_format=torch.preserve_format)
                shadows = _ptr_array([self.shadow[p] for p in gp])
            plan["groups"].append({
                "group": group, "idx": idx, "n": len(gp), "p": _ptr_array(gp),
                "m": _ptr_array([states[i]["exp_avg"] for i in idx]), "v": _ptr_array([states[i]["exp_avg_sq"] for i in idx]),
                "shadow": shadows, "numel": (ctypes.c_int64 * len(gp))(*[p.numel() for p in gp]),
            })
        self._plans = {key: plan}  # keep the latest only: it holds references to every state tensor
        return plan

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        active = [(g, p) for g in self.param_groups for p in g["params"] if p.grad is not None]
        if not active:
            return loss
        device = active[0][1].device
        plan = self._plan(active, device)
        params, states = plan["params"], plan["states"]
        grads = []
        for p in params:
            g = p.grad
            if g.dtype is not torch.float32 or g.is_sparse or g.device != device or g.stride() != p.stride():
                raise NotImplementedError(f"FusedClipAdam: gradient must be dense fp32 with the parameter's layout, got {g.dtype}, "
                                          f"strides {tuple(g.stride())} vs {tuple(p.stride())}")
            grads.append(g)
        L = _lib.lib()
        with _lib.device_guard(device):
            stream = _lib.stream_ptr(device)
            # The kernels keep one step counter (the first parameter's, advanced by the first pass); torch keeps one
            # per parameter, all equal, and a checkpoint must hold them as separate tensors: the others are advanced
            # by one multi-tensor add.
            step = states[0]["step"]
            fresh = self.__dict__.get("_fresh_step")
            if fresh is not None:
                fresh[1] = True  # stepped: parameters that join later get a counter of their own
            if plan["others"]:
                torch._foreach_add_(plan["others"], 1.0)
            nslots = plan["nslots"]
            if self._slots is None or self._slots.numel() < nslots or self._slots.device != device:
                self._slots = torch.empty(nslots, dtype=torch.float32, device=device)
            if self.grad_norm is None or self.grad_norm.device != device:
                self.grad_norm = torch.zeros((), dtype=torch.float32, device=device)
            # one squared-norm pass over every gradient (the norm is global, as in clip_grad_norm_)
            g_all = _ptr_array(grads)
            _lib.check(L.sfh_adam_grad_sumsq(len(params), g_all, plan["numel"], _lib.ptr(self._slots), _lib.ptr(step), stream),
                       "FusedClipAdam (gradient norm)")
            # one update per hyperparameter group (usually one); each folds ALL slots
            for gpl in plan["groups"]:
                group = gpl["group"]
                desc = AdamDesc(group["lr"], group["betas"][0], group["betas"][1], group["eps"], group["weight_decay"],
                                -1.0 if self.max_norm is None else float(self.max_norm),
                                -1 if self.shadow_dtype is None else _lib.dtype_code(self.shadow_dtype))
                g_arr = g_all if len(plan["groups"]) == 1 else _ptr_array([grads[i] for i in gpl["idx"]])
                rc = L.sfh_adam_clip_step(ctypes.byref(desc), gpl["n"], gpl["p"], g_arr, gpl["m"], gpl["v"], gpl["shadow"], gpl["numel"],
                                          _lib.ptr(self._slots), nslots, _lib.ptr(step), _lib.ptr(self.grad_norm), stream)
                _lib.check(rc, "FusedClipAdam (update)")
            if self.shadow_dtype is not None:
                for p in params:  # the kernel wrote parameter and copy together
                    p._sfh_shadow = self.shadow[p]
                    p._sfh_shadow_version = p._version
            self._refresh_packs(params)
        return loss

    def _refresh_packs(self, params):
        """Packed forms of convolution weights that the modules keep on the parameters (``p._sfh_packs``) are derived
        from what this step just wrote: they are packed again here, all in one batch, and stamped as current."""
        from . import conv3d as _c3
        plan = self._pack_plan
        if plan is None or plan[0] != _c3.PackedWeights.generation or plan[1] is not params:
            pairs = []
            for p in params:
                table = p.__dict__.get("_sfh_packs")
                if table:
                    src = self.shadow.get(p) if self.shadow_dtype is not None else p
                    pairs.extend((p, e) for e in table.values() if e and e.source is src)
            batch = _c3._PackBatchPlan([e for _, e in pairs]) if pairs else None
            plan = self._pack_plan = (_c3.PackedWeights.generation, params, pairs, batch)
        _, _, pairs, batch = plan
        if batch is not None:
            batch.run()
            for p, e in pairs:
                e.version = p._version
                e.maintained = True

    def state_dict(self):
        """As ``torch.optim.Optimizer.state_dict``; every parameter's ``step`` is a tensor of its own there (inside the
        optimizer the parameters share one), so that a consumer which advances them one by one -- ``torch.optim.Adam``
        after ``load_state_dict`` -- counts right."""
        sd = super().state_dict()
        sd["state"] = {k: (dict(v, step=v["step"].clone()) if torch.is_tensor(v.get("step")) else v) for k, v in sd["state"].items()}
        return sd

    def load_state_dict(self, state_dict):
        """As ``torch.optim.Optimizer.load_state_dict``, then the state is brought into the form the kernels read.

        torch leaves ``step`` wherever the checkpoint held it (a host tensor after the reference's restore path,
        ``ScaFFold/utils/checkpointing.py:309-340``, and in every checkpoint of a non-fused ``torch.optim.Adam``) and keeps
        the strides the moments were saved with. The kernels dereference ``step`` on the device and walk parameter,
        gradient and both moments as one flat array, so here ``step`` becomes a 0-dim fp32 tensor on the parameter's
        device and the moments are re-laid out to the parameter's own strides (values follow their logical index)."""
        super().load_state_dict(state_dict)
        self._plans = {}  # the state tensors were replaced
        self._pack_plan = None
        steps = set()
        for group in self.param_groups:
            for p in group["params"]:
                st = self.state.get(p)
                if not st:
                    continue
                missing = [k for k in ("step", "exp_avg", "exp_avg_sq") if k not in st]
                if missing:
                    raise NotImplementedError(f"FusedClipAdam: loaded state lacks {missing} (amsgrad / foreign optimizers are not served)")
                step = st["step"]
                step = step.detach() if torch.is_tensor(step) else torch.tensor(float(step))
                steps.add(float(step))  # a load is not the hot loop: one host read per parameter
                st["step"] = step.to(device=p.device, dtype=torch.float32).reshape(()).clone()
                for k in ("exp_avg", "exp_avg_sq"):
                    st[k] = self._like_param(p, st[k], k)
        if len(steps) > 1:
            raise NotImplementedError(f"FusedClipAdam: the kernels keep one step counter for all parameters, the loaded state has {sorted(steps)}")
        # all equal: one tensor serves every parameter again
        shared = None
        for group in self.param_groups:
            for p in group["params"]:
                st = self.state.get(p)
                if st:
                    if shared is None or shared.device != st["step"].device:
                        shared = st["step"]
                    st["step"] = shared
        self._fresh_step = None

    @staticmethod
    def _like_param(p, t, what):
        """``t`` as an fp32 tensor on ``p``'s device with ``p``'s strides (no copy when it already is)."""
        if not torch.is_tensor(t) or t.shape != p.shape:
            raise ValueError(f"FusedClipAdam: loaded {what} has shape {tuple(getattr(t, 'shape', ()))}, the parameter {tuple(p.shape)}")
        if t.device == p.device and t.dtype is torch.float32 and t.stride() == p.stride():
            return t
        out = torch.empty_like(p, dtype=torch.float32, memory_format=torch.preserve_format)
        out.copy_(t)
        return out

    def _check_state(self, p, st):
        """What the kernels assume about a parameter's state; raises rather than hand the device a host address or a
        permuted moment."""
        step = st["step"]
        if not torch.is_tensor(step) or step.device != p.device or step.dtype is not torch.float32 or step.numel() != 1:
            raise NotImplementedError(f"FusedClipAdam: step must be a one-element fp32 tensor on {p.device}, got "
                                      f"{getattr(step, 'dtype', type(step))} on {getattr(step, 'device', 'the host')}; "
                                      "load checkpoints through load_state_dict")
        for k in ("exp_avg", "exp_avg_sq"):
            t = st[k]
            if t.device != p.device or t.dtype is not torch.float32 or t.shape != p.shape or t.stride() != p.stride():
                raise NotImplementedError(f"FusedClipAdam: {k} must be fp32 on {p.device} with the parameter's strides {tuple(p.stride())}, "
                                          f"got {t.dtype} on {t.device} with strides {tuple(t.stride())}")

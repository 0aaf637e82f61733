"""Host layer: ``torch.optim.Optimizer`` classes with HeavyBall's constructor signatures and observable behaviour,
whose ``step()`` runs on the HIP kernels of libhbstep.so.

What is mirrored from the reference (HomebrewML/HeavyBall 3.2.0), by observable behaviour only:

  * keyword handling and errors: heavyball/chainable.py:197-220 (``_build_defaults``)
  * param-group contents: heavyball/chainable.py:2387-2408, heavyball/utils.py:1506-1525
  * the step loop: heavyball/utils.py:1815-1834, heavyball/chainable.py:2510-2570 (step counter as an int64 0-d tensor,
    lr warm-up as an fp32 0-d tensor, gradients consumed, ``group["step"]`` reset to None, lr restored)
  * state layout: ``state[p][0][f"{fn}_{name}_{idx}"]`` with ``"::ecc"`` siblings, ``"param::ecc"``, ``"is_initialized"``
    and ``"step"`` (heavyball/chainable.py:73-74, :254-258, :2442, :2559; heavyball/utils.py:1554-1563)
  * ``state_dict()`` extras: heavyball/utils.py:1527-1549, heavyball/chainable.py:2410-2415, :2452-2484
  * ``param_ecc`` narrows the live parameter at construction: heavyball/chainable.py:2421-2444

What is different by design: parameters and optimizer state of a group live in one slab (heavyball_amd/slab.py); the
tensors in ``optimizer.state`` and ``param.data`` are views into it, and one kernel launch updates the whole group.
"""

import io
import math
import pickle
import warnings
from typing import Dict, List, Optional, Tuple

import numpy as np
import torch

from . import _lib
from .slab import Slab

use_default = object()

_INSTANCE_ATTRS = (
    "compile_step",
    "finite_differences",
    "fallback_to_finite_differences",
    "hvp_interval",
    "hessian_approx",
    "consume_grad",
)
_PASSTHROUGH_KWARGS = frozenset({"orig_shapes", *_INSTANCE_ATTRS})
_RENAMED_KWARGS = {"foreach": "multi_tensor"}
_REMOVED_KWARGS = frozenset({"stochastic_schedule", "normalize_grads", "correct_bias", "inverse_free", "adaptive"})

_ECC_DTYPES = {
    "bf16+8": (torch.bfloat16, torch.int8),
    "bf16+16": (torch.bfloat16, torch.int16),
    "fp16+8": (torch.float16, torch.int8),
    "fp16+16": (torch.float16, torch.int16),
}
_PLAIN_FMT = {torch.float32: _lib.FMT_F32, torch.bfloat16: _lib.FMT_BF16, torch.float16: _lib.FMT_F16}

_warned = set()


def warn_once(msg):
    if msg not in _warned:
        warnings.warn(msg)
        _warned.add(msg)


def build_defaults(locals_dict):
    """heavyball/chainable.py:197-220: split ``locals()`` of a constructor into (params, defaults)."""
    d = locals_dict.copy()
    d.pop("self", None)
    d.pop("__class__", None)
    params = d.pop("params")
    kwargs = d.pop("kwargs")
    for old, new in _RENAMED_KWARGS.items():
        if old in kwargs:
            warnings.warn(f"'{old}' was renamed to '{new}' in HeavyBall 3.0. Pass '{new}' instead.", FutureWarning, stacklevel=4)
            d[new] = kwargs.pop(old)
    hit = _REMOVED_KWARGS & kwargs.keys()
    if hit:
        raise TypeError(f"Removed in HeavyBall 3.0: {', '.join(sorted(hit))}. See docs/heavyball3.md for migration details.")
    unknown = kwargs.keys() - _PASSTHROUGH_KWARGS
    if unknown:
        raise TypeError(f"unknown keyword arguments: {sorted(unknown)}")
    d.update(kwargs)
    return params, d


def f32(x) -> torch.Tensor:
    """A python float as the fp32 0-d tensor the reference's ``scalar_guard`` makes (heavyball/utils.py:1093-1094)."""
    if isinstance(x, torch.Tensor):
        return x.detach().to(dtype=torch.float32, device="cpu")
    return torch.empty((), dtype=torch.float32).fill_(x)


def beta_debias(beta: torch.Tensor, step: torch.Tensor) -> torch.Tensor:
    """heavyball/utils.py:337-338 on fp32 / int64 0-d tensors."""
    return 1 - (1 - beta) / (1 - beta**step)


def lerp_weights(beta_debiased: torch.Tensor) -> Tuple[float, float]:
    """(a, 1 - a) with a = 1 - beta', each rounded to fp32 as in heavyball/utils.py:1847 and :1048."""
    a = 1 - beta_debiased
    return float(a), float(1 - a)


def mars_weights(group) -> Tuple[float, float]:
    """(a, 1 - a) of MARS' stochastic lerp.  heavyball/chainable.py:645 passes (mars_gamma, beta1) into (beta1, gamma) of
    heavyball/utils.py:3623, so the weight is -beta1 * mars_gamma / (1 - mars_gamma)."""
    b1m, gam = group["mars_gamma"], (group["betas"][0] if group.get("beta") is None else group["beta"])
    am = f32(-gam * b1m / (1 - b1m))
    return float(am), float(1 - am)


def debiased_weights(beta: torch.Tensor, step) -> Tuple[float, float]:
    """``lerp_weights(beta_debias(beta, step))`` for an fp32 0-d ``beta``, at a fraction of the host time: the power is
    torch's own (its rounding belongs to the library), the subtractions and the division are single IEEE fp32
    operations and run on numpy scalars, where each costs a tenth of a microsecond instead of several."""
    one = np.float32(1)
    b, power = np.float32(beta.item()), np.float32((beta**step).item())
    with np.errstate(all="ignore"):
        a = one - (one - (one - b) / (one - power))
        return float(a), float(one - a)


_ONE32 = np.float32(1)


def debiased_weights_np(beta: float, n: int) -> Tuple[float, float]:
    """``debiased_weights`` for a python-float beta and a python-int step, on numpy scalars throughout.  The power of a 0-d fp32
    tensor by a 0-d int64 tensor is the C library's ``powf`` on the CPU, and so is numpy's ``float32 ** float32``
    (tests/test_host_logic.py compares the two over many steps), which makes the whole chain a handful of 0.1-microsecond operations."""
    b = np.float32(beta)
    with np.errstate(all="ignore"):
        a = _ONE32 - (_ONE32 - (_ONE32 - b) / (_ONE32 - b ** np.float32(n)))
        return float(a), float(_ONE32 - a)


def step_lr_np(base_lr: float, n: int, warmup_steps: int) -> np.float32:
    """``base_lr * step / step.clamp(min=warmup_steps + 1)`` of heavyball/chainable.py:2560 with ``step`` an int64 0-d tensor: the
    python float is rounded to fp32, the product and the quotient are single fp32 operations."""
    return np.float32(base_lr) * np.float32(n) / np.float32(max(n, warmup_steps + 1))


_hostloop_module = False  # False: not looked for yet; None: not built


def hostloop():
    """The C++ helper of the cached-plan step (csrc/hostloop.cpp, built next to libhbstep.so), or None when it has not been built:
    the step then walks its tensors in Python, with the same checks."""
    global _hostloop_module
    if _hostloop_module is False:
        import importlib.util
        import os

        path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "_hostloop.so")
        _hostloop_module = None
        if os.path.exists(path):
            spec = importlib.util.spec_from_file_location("_hostloop", path)
            mod = importlib.util.module_from_spec(spec)
            spec.loader.exec_module(mod)
            _hostloop_module = mod
    return _hostloop_module


def current_stream_ptr(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


class _Unpickle(pickle.Unpickler):
    """``precond_schedule`` travels as pickled bytes (heavyball/utils.py:1534); only plain numbers/None are accepted."""

    def find_class(self, module, name):
        raise pickle.UnpicklingError("only plain values are accepted for precond_schedule")


class Bucket:
    """Same-device, same-dtype parameters of one group, with their slab."""

    def __init__(self, params: List[torch.nn.Parameter], param_dtype: torch.dtype):
        self.params = params
        self.index = {id(p): i for i, p in enumerate(params)}
        self.device = params[0].device
        self.param_dtype = param_dtype
        self.slab = Slab([p.shape for p in params], self.device)
        self.counts = None  # caution scratch
        self.grad_tables: Dict[Tuple, Tuple[torch.Tensor, torch.Tensor]] = {}
        self._home = None
        self.state_ready = {}  # state layout key -> indices of the tensors whose state entries exist

    def caution_scratch(self) -> torch.Tensor:
        if self.counts is None:
            self.counts = torch.zeros(len(self.params) * _lib.CAUTION_SLOTS, dtype=torch.int32, device=self.device)
        return self.counts

    def grad_ptr_table(self, key, ptrs: List[int]) -> torch.Tensor:
        """Device array of per-tensor gradient pointers (indexed by slab tensor index).  Gradient buffers usually come back
        at the addresses of a few steps ago (the caching allocator, or a handful of buffers in rotation), so the last
        few tables are kept and one is uploaded only for a set of pointers not seen among them."""
        tup = (key, *ptrs)
        hit = self.grad_tables.get(tup)
        if hit is not None:
            return hit[0]
        host = torch.tensor(ptrs, dtype=torch.int64)
        if self.device.type == "cuda":
            host = host.pin_memory()
        dev = host.to(self.device, non_blocking=True)
        if len(self.grad_tables) >= 16:
            self.grad_tables.pop(next(iter(self.grad_tables)))  # oldest first; a kernel in flight keeps its table through _last_launch
        self.grad_tables[tup] = (dev, host)
        return dev

    def grad_ptr_table_from(self, key, ptrs: torch.Tensor) -> torch.Tensor:
        """``grad_ptr_table`` for pointers that already sit in an int64 CPU tensor; ``key``: (gradient dtype, the tensor's bytes)."""
        hit = self.grad_tables.get(key)
        if hit is not None:
            return hit[0]
        host = ptrs.clone().pin_memory() if self.device.type == "cuda" else ptrs.clone()
        dev = host.to(self.device, non_blocking=True)
        if len(self.grad_tables) >= 16:
            self.grad_tables.pop(next(iter(self.grad_tables)))
        self.grad_tables[key] = (dev, host)
        return dev

    def home_ptrs(self) -> List[int]:
        """Address of every parameter's view of the slab: what ``p.data_ptr()`` must be while the slab backs ``p``."""
        if self._home is None:
            base, size = self.slab.ptr("param"), self.slab.roles["param"].element_size()
            self._home = [base + int(o) * size for o in self.slab.offsets_np]
        return self._home


class HBOptimizer(torch.optim.Optimizer):
    """Common runtime of the MI355X optimizers (the observable behaviour of StatefulOptimizer + ChainOpt + BaseOpt)."""

    ema_decay: float = 0.001
    compile_step: bool = False
    hessian_approx: bool = False
    precond_schedule = None
    finite_differences: bool = False
    fallback_to_finite_differences: bool = True
    _fallback_enabled: bool = False
    hvp_interval: int = 1
    consume_grad: bool = True
    promote: bool = False
    palm: bool = False

    #: "philox" (counter-based stochastic rounding) or "half" (deterministic: every stochastic site rounds half up)
    rounding: str = "philox"
    #: with MARS, write the corrected gradient back into the gradient buffer as the reference does (chainable.py:646);
    #: off by default because ``step()`` drops the gradient right after (consume_grad) and the write costs bandwidth
    mars_write_grad: bool = False

    global_defaults = {"caution": False, "lr": 1, "warmup_steps": 0, "weight_decay": 0, "eps": 1e-8}  # chainable.py:2387-2393

    def __init__(self, params, defaults, gradient_clipping=use_default, update_clipping=use_default, palm=use_default,
                 compile_step=use_default, promote=use_default):  # fmt: skip
        defaults = dict(defaults)
        defaults.pop("orig_shapes", None)
        cs = defaults.pop("compile_step", use_default)
        self.compile_step = self._pick(self._pick(compile_step, cs), self.compile_step)
        pr = defaults.pop("promote", use_default)
        self.promote = self._pick(self._pick(promote, pr), self.promote)
        defaults.pop("update_clipping", None)
        defaults.pop("gradient_clipping", None)
        self.gradient_clipping = self._resolve_clip(self._pick(gradient_clipping, None))
        self.update_clipping = self._resolve_clip(self._pick(update_clipping, None))
        self._use_palm = bool(self._pick(palm, self.palm))
        for attr in _INSTANCE_ATTRS:
            if attr in defaults:
                val = defaults.pop(attr)
                if val is not use_default:
                    setattr(self, attr, val)
        base = dict(self.global_defaults)
        base.update({k: v for k, v in defaults.items() if v is not use_default})
        base.setdefault("multi_tensor", True)
        self._buckets: Dict[int, List[Bucket]] = {}
        self._loc: Dict[int, Tuple[Bucket, int]] = {}  # id(parameter) -> (bucket, index in the bucket)
        self._plans: Dict[int, "_StepPlan"] = {}  # group index -> cached launch plan of the fused step (FirstOrder._fast_step)
        self.rng_seed = int(torch.initial_seed()) & 0xFFFFFFFFFFFFFFFF
        self.use_ema = False
        self.inner_group = {}
        self._is_preconditioning = None
        super().__init__(params, base)
        for gi, group in enumerate(self.param_groups):
            self._adopt_group(gi, group)

    # -- construction -------------------------------------------------------------------------------------------
    def _betas(self, group, step):
        beta1 = group["betas"][0] if group.get("beta") is None else group["beta"]
        if self._use_palm:  # heavyball/chainable.py:1921-1925
            beta2 = 1 - group["step"] ** -group["beta2_scale"]
            group["betas"] = (beta1, beta2, *group["betas"][2:])
        else:
            beta2 = group["betas"][1]
        return f32(beta1), f32(beta2)

    @staticmethod
    def _pick(a, b):
        return b if a is use_default else a

    @staticmethod
    def _resolve_clip(fn):
        if fn is None:
            return None
        from . import clipping

        return clipping.resolve(fn)

    def add_param_group(self, param_group):
        super().add_param_group(param_group)
        if hasattr(self, "_plans"):
            self._plans.clear()
        if hasattr(self, "_buckets"):
            gi = len(self.param_groups) - 1
            if gi not in self._buckets and getattr(self, "_constructed", False):
                self._adopt_group(gi, self.param_groups[gi])

    def _adopt_group(self, gi: int, group: dict):
        """Move the group's parameters into slabs (and narrow them under param_ecc, chainable.py:2421-2444)."""
        self._constructed = True
        for key in ("ecc", "param_ecc"):
            mode = group.get(key)
            if mode and mode not in _ECC_DTYPES:
                raise KeyError(mode)
        storage = group.get("storage_dtype", "float32")
        if not group.get("ecc") and getattr(torch, storage) not in (torch.float32, torch.bfloat16):
            raise NotImplementedError(f"storage_dtype={storage!r}: the kernels store optimizer state as float32, bfloat16 or an ECC pair")
        pecc = group.get("param_ecc")
        by_key: Dict[Tuple, List] = {}
        for p in group["params"]:
            dt = _ECC_DTYPES[pecc][0] if pecc else p.dtype
            if dt not in (torch.float32, torch.bfloat16) and not pecc:
                raise NotImplementedError(f"parameters of dtype {p.dtype} are not supported (float32, bfloat16, or param_ecc)")
            by_key.setdefault((p.device, dt, self._route(p)), []).append(p)
        buckets = []
        for (device, dt, _), plist in by_key.items():
            b = Bucket(plist, dt)
            buf_dtype = dt
            b.slab.role("param", buf_dtype)
            if pecc:
                b.slab.role("param::ecc", _ECC_DTYPES[pecc][1])
            for i, p in enumerate(plist):
                view = b.slab.view("param", i)
                if pecc and p.dtype != dt:
                    self._encode_param(b, i, p.data.float().contiguous(), group)
                else:
                    view.copy_(p.data)
                p.data = view
                if pecc:
                    self._state0(p)["param::ecc"] = b.slab.view("param::ecc", i)
            buckets.append(b)
            for i, p in enumerate(plist):
                self._loc[id(p)] = (b, i)
        self._buckets[gi] = buckets

    def _route(self, p) -> int:
        """Parameters that take different transforms (heavyball/chainable.py:169-170 ``route``) get slabs of their own,
        so that each slab only carries the state roles its transform needs."""
        return 0

    def _encode_param(self, b: Bucket, i: int, fp32: torch.Tensor, group: dict):
        """ECCConfig.init_correction (chainable.py:240-241): primary = RNE(fp32), correction from the residual."""
        if b.device.type != "cuda":
            raise _lib.HbError("param_ecc needs the parameters on a GPU: the ECC encode runs in libhbstep.so")
        L = _lib.lib()
        prim, corr = b.slab.view("param", i), b.slab.view("param::ecc", i)
        with torch.cuda.device(b.device):
            rc = L.hb_ecc_encode(fp32.data_ptr(), prim.data_ptr(), corr.data_ptr(), fp32.numel(), _lib.ECC_FMT[group["param_ecc"]],
                                 self._rng_mode(), self.rng_seed, 0, _lib.STREAM_INIT_PARAM, int(b.slab.offsets_np[i]),
                                 current_stream_ptr(b.device))  # fmt: skip
        _lib.check(rc, "hb_ecc_encode")

    def _rng_mode(self) -> int:
        if self.rounding == "philox":
            return _lib.RNG_PHILOX
        if self.rounding == "half":
            return _lib.RNG_HALF
        raise ValueError(f"rounding must be 'philox' or 'half', not {self.rounding!r}")

    # -- state ---------------------------------------------------------------------------------------------------
    def _state0(self, p) -> dict:
        return self.state[p].setdefault(0, {})

    def state_(self, p, fail: bool = True) -> dict:
        """heavyball/utils.py:1554-1563."""
        if p not in self.state and not any(p is q for g in self.param_groups for q in g["params"]):
            if not fail:
                return {}
            raise KeyError("Tensor has no tracked state.")
        return self._state0(p)

    def state_size(self) -> int:
        """heavyball/utils.py:1635-1647: bytes held by optimizer state tensors."""
        total, seen = 0, set()
        for st in self.state.values():
            for d in st.values():
                if isinstance(d, dict):
                    for v in d.values():
                        if isinstance(v, torch.Tensor) and id(v) not in seen:
                            seen.add(id(v))
                            total += v.numel() * v.element_size()
        return total

    def _find_bucket(self, gi: int, p) -> Tuple[Bucket, int]:
        loc = self._loc.get(id(p))
        if loc is None or loc[0].params[loc[1]] is not p:
            raise KeyError("Tensor has no tracked state.")
        return loc

    def _check_home(self, b: Bucket, items):
        """``step()`` updates the slab, so ``p.data`` must still be the slab's view of ``p``.  A parameter whose data was
        rebound since (``model.bfloat16()``, ``p.data = ...``, a swap of averaged weights) is moved back: its current
        values are copied into the slab and ``p.data`` is pointed there again, as after ``load_state_dict``.
        ``items``: [(index, parameter, ...)]."""
        home = b.home_ptrs()
        for it in items:
            i, p = it[0], it[1]
            if p.data_ptr() != home[i] and p.numel():
                view = b.slab.view("param", i)
                if p.device != b.device:
                    raise _lib.HbError("a parameter was moved to another device after the optimizer was constructed")
                if p.dtype != view.dtype:
                    raise _lib.HbError(f"a parameter changed its dtype from {view.dtype} to {p.dtype} after the optimizer was constructed; "
                                       "construct the optimizer after casting the model")  # fmt: skip
                view.copy_(p.data)
                p.data = view

    # -- step ----------------------------------------------------------------------------------------------------
    def _schedule_tick(self):
        """heavyball/utils.py:1816-1819 and :3494-3500: float-accumulated preconditioning schedule."""
        if self.precond_schedule is None:
            self._is_preconditioning = False
            return
        g = self.inner_group
        g["cumulative_prob_prob_step"] = g.get("cumulative_prob_prob_step", 0) + 1
        prob = self.precond_schedule
        if not isinstance(prob, float):
            prob = prob(g["cumulative_prob_prob_step"])
        cumulative = g.get("cumulative_prob", 0)
        g["cumulative_prob"] = cumulative + prob
        self._is_preconditioning = int(g["cumulative_prob"]) > int(cumulative)

    def step(self, closure=None):
        self._schedule_tick()
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        with torch.no_grad():
            for gi, group in enumerate(self.param_groups):
                if "param_count" not in group:
                    group["param_count"] = sum(p.numel() for p in group["params"])
                group["is_preconditioning"] = self._is_preconditioning
                self._step(gi, group)
        return loss

    def _fast_step(self, gi: int, group: dict) -> bool:
        """A step from a cached launch plan; False when there is none or it does not fit this step (the general path runs then)."""
        return False

    @staticmethod
    def _note_lr(group: dict):
        """heavyball/chainable.py:2542-2551: the learning rate the group is stepped with is remembered; a change is reported once."""
        if "base_lr" not in group:
            group["base_lr"] = group["lr"]
        elif group["base_lr"] != group["lr"]:
            warn_once(
                f"Learning rate changed between steps. This is an experimental feature and "
                f"only supported with multi_tensor=True (currently multi_tensor={group['multi_tensor']})."
            )
            group["base_lr"] = group["lr"]

    def _step(self, gi: int, group: dict):
        """heavyball/chainable.py:2510-2570."""
        if gi in self._plans and self._fast_step(gi, group):
            return
        if gi not in self._buckets:
            self._adopt_group(gi, group)
        self._note_lr(group)
        caution = group["caution"]
        active = []
        for p in group["params"]:
            g = p.grad
            if g is None:
                continue
            if self.consume_grad:
                p.grad = None
            active.append((p, g))
        if not active:
            return
        step = group.get("_group_step")
        if step is None:
            for p in group["params"]:
                st = self.state.get(p)
                if not isinstance(st, dict):
                    continue
                for idx_state in st.values():
                    if isinstance(idx_state, dict) and "step" in idx_state:
                        step = idx_state["step"]
                        break
                if step is not None:
                    break
            else:
                step = 0
        if isinstance(step, torch.Tensor):
            step = step.detach().to(device="cpu", dtype=torch.int64)
        else:
            step = torch.empty((), dtype=torch.int64).fill_(step)
        group["_group_step"] = group["step"] = step = step + 1
        self._state0(active[0][0])["step"] = step
        group["prev_lr"] = group["lr"] = group["base_lr"] * step / step.clamp(min=group["warmup_steps"] + 1)
        try:
            self._run_group(gi, group, active)
        finally:
            group["caution"] = caution
            group["lr"] = group["base_lr"]
            group["step"] = None

    def _clip_role(self, L, kind, role_name, buckets):
        """The clip functions of heavyball/utils.py:3226-3297 applied in place to an fp32 slab role: per-tensor sums of
        squares (``hb_sumsq``), the scale ``clip_at / max(norm, clip_at, eps)`` per tensor or for the whole group, then
        ``hb_scale``.  ``buckets``: [(bucket, sorted tensor indices)].  Returns what must stay alive until the stream is done."""
        clip_at, eps = 1.0, 1e-8
        sums, plan = [], []
        for b, act in buckets:
            role = b.slab.role(role_name, torch.float32)
            chunks, n_chunks = b.slab.chunks(tuple(act))
            offsets, numel = b.slab.meta()
            partial = torch.zeros(max(n_chunks, 1), dtype=torch.float64, device=b.device)
            out = torch.zeros(len(b.params), dtype=torch.float64, device=b.device)
            with torch.cuda.device(b.device):
                _lib.check(L.hb_sumsq(role.data_ptr(), _lib.FMT_F32, offsets.data_ptr(), numel.data_ptr(), chunks.data_ptr(), n_chunks,
                                      len(b.params), partial.data_ptr(), out.data_ptr(), current_stream_ptr(b.device)), "hb_sumsq")  # fmt: skip
            sums.append(out)
            plan.append((b, act, chunks, n_chunks, offsets, numel, role, partial))
        floor = max(clip_at, eps)
        if kind in ("global_l2norm_clip", "global_rmsnorm_clip"):  # one norm over every tensor of the group
            total = sum(o.sum().to(sums[0].device) for o in sums)
            count = sum(int(b.slab.numels[i]) for b, act in buckets for i in act)
            norm = (total / count if kind == "global_rmsnorm_clip" else total).sqrt().to(torch.float32)
            scales = [(clip_at / norm.clamp(min=floor)).reshape(1).to(b.device) for b, *_ in plan]
            per_tensor = 0
        else:
            scales = []
            for (b, *_rest), o in zip(plan, sums):
                _, numel = b.slab.meta()
                sq = o / numel.clamp(min=1).to(torch.float64) if kind == "rmsnorm_clip_" else o
                scales.append((clip_at / sq.sqrt().to(torch.float32).clamp(min=floor)).contiguous())
            per_tensor = 1
        for (b, act, chunks, n_chunks, offsets, numel, role, _), sc in zip(plan, scales):
            with torch.cuda.device(b.device):
                _lib.check(L.hb_scale(role.data_ptr(), sc.data_ptr(), per_tensor, offsets.data_ptr(), numel.data_ptr(), chunks.data_ptr(),
                                      n_chunks, current_stream_ptr(b.device)), "hb_scale")  # fmt: skip
        return plan, scales

    def _mars_prologue(self, L, group, b, lst, gdt, step, mars_a, mars_oma, state_fmt, k_o):
        """MARS alone over one bucket: ``mars_old_grad`` takes the raw gradients, the corrected ones (rounded to the gradient
        dtype) land in the fp32 slab role ``_clip``."""
        offsets, numel = b.slab.meta()
        chunks, n_chunks = b.slab.chunks(tuple(i for i, _ in lst))
        ptrs = [0] * len(b.params)
        for i, g in lst:
            ptrs[i] = g.data_ptr()
        table = b.grad_ptr_table(gdt, ptrs)
        out = b.slab.role("_clip", torch.float32)
        d = _lib.HbStepDesc()
        d.param, d.param_fmt = out.data_ptr(), _lib.FMT_F32
        d.grad, d.grad_ptrs, d.grad_fmt = None, table.data_ptr(), _PLAIN_FMT[gdt]
        d.old_grad, d.old_grad_corr, d.state_fmt = b.slab.ptr(k_o), b.slab.ptr(k_o + "::ecc"), state_fmt
        d.offsets, d.numel, d.chunks = offsets.data_ptr(), numel.data_ptr(), chunks.data_ptr()
        d.n_chunks, d.n_tensors = n_chunks, len(b.params)
        d.algo, d.flags = _lib.ALGO_ADAM, _lib.FLAG_MARS | _lib.FLAG_MARS_ONLY  # the prologue is the same for every algorithm
        d.mars_a, d.one_minus_mars_a = mars_a, mars_oma
        d.rng_mode, d.step, d.seed = self._rng_mode(), int(step) & 0xFFFFFFFF, self.rng_seed
        with torch.cuda.device(b.device):
            _lib.check(L.hb_fused_step(d, current_stream_ptr(b.device)), "hb_fused_step (MARS prologue)")
        self._last_launch = (d, (table, chunks, offsets, numel))

    def _run_gen(self, gen):
        """Runs a step generator to its end.  Such a generator yields ``(clip kind, slab role, [(bucket, tensor indices)])`` wherever
        the chain clips by a norm, and is sent back what ``_clip_role`` returns; its own return value is handed on."""
        L = _lib.lib()
        try:
            req = next(gen)
            while True:
                req = gen.send(self._clip_role(L, req[0], req[1], req[2]))
        except StopIteration as done:
            return done.value

    def _run_gens(self, gens):
        """Several step generators side by side (the routes of one parameter group): they reach their clip points in the same
        order, and each point is clipped once over the tensors of all of them, so that a norm over the whole group is one norm."""
        L = _lib.lib()
        waiting = []
        for g in gens:
            try:
                waiting.append((g, next(g)))
            except StopIteration:
                pass
        while waiting:
            kind, role = waiting[0][1][0], waiting[0][1][1]
            if any(r[0] != kind or r[1] != role for _, r in waiting):
                raise _lib.HbError("the routes of a parameter group reached different clip points")
            keep = self._clip_role(L, kind, role, [bk for _, r in waiting for bk in r[2]])
            nxt = []
            for g, _ in waiting:
                try:
                    nxt.append((g, g.send(keep)))
                except StopIteration:
                    pass
            waiting = nxt

    def _clip_gradients(self, L, group, buckets, step, gathered=False):
        return self._run_gen(self._clip_gradients_gen(L, group, buckets, step, gathered))

    def _clip_gradients_gen(self, L, group, buckets, step, gathered=False):
        """``gradient_clipping`` (heavyball/chainable.py:2696-2699): the gradients of the group are gathered into the fp32
        slab role ``_clip``, clipped there (a clip point, see ``_run_gen``) and, for 16-bit gradients, rounded back the way
        ``copy_stochastic_`` does (bf16: ``hb_sr_bf16``; fp16: a cast).  ``buckets``: [(bucket, [(index, gradient)], gradient dtype)].  Returns,
        per bucket, the slab role and format the step then reads its gradients from.  Three extra passes over the
        gradients: a capability, not a tuned path."""
        for b, lst, gdt in buckets:
            b.slab.role("_clip", torch.float32)
            if not gathered:  # otherwise an earlier pass (MARS) has left the gradients in the role
                for i, g in lst:
                    b.slab.view("_clip", i).copy_(g)
        keep = None
        if self.gradient_clipping is not None:  # None: the caller only wants the gathered role in the gradients' dtype
            keep = yield (self.gradient_clipping, "_clip", [(b, [i for i, _ in lst]) for b, lst, _ in buckets])
        result = []
        for b, lst, gdt in buckets:
            role = b.slab.role("_clip", torch.float32)
            if gdt == torch.bfloat16:
                narrow = b.slab.role("_clip16", torch.bfloat16)
                with torch.cuda.device(b.device):
                    _lib.check(L.hb_sr_bf16(role.data_ptr(), narrow.data_ptr(), role.numel(), self._rng_mode(), self.rng_seed,
                                            int(step) & 0xFFFFFFFF, _lib.STREAM_CLIP, 0, current_stream_ptr(b.device)), "hb_sr_bf16")  # fmt: skip
                result.append((narrow, torch.bfloat16, keep))
            elif gdt == torch.float16:
                # a float16 buffer takes the clipped values through a plain cast (heavyball/utils.py:2363-2370 rounds stochastically
                # into bfloat16 only); per tensor, since the bucket may hold tensors with gradients of another dtype
                b.slab.role("_clip16h", torch.float16)
                for i, _ in lst:
                    b.slab.view("_clip16h", i).copy_(b.slab.view("_clip", i))
                result.append((b.slab.role("_clip16h", torch.float16), torch.float16, keep))
            else:
                result.append((role, torch.float32, keep))
        return result

    def _clip_updates(self, L, buckets):
        """``update_clipping`` (heavyball/chainable.py:2700-2701) for optimizers whose update sits in the fp32 slab role
        ``_update`` before ``hb_update_param`` (Muon, SOAP).  ``buckets``: [(bucket, sorted tensor indices)]."""
        return self._clip_role(L, self.update_clipping, "_update", buckets)

    def _run_group(self, gi, group, active):
        raise NotImplementedError

    # -- checkpointing ---------------------------------------------------------------------------------------------
    def state_dict(self):
        sd = super().state_dict()
        for g in sd["param_groups"]:
            for k in [k for k in g if k.startswith("_")]:
                del g[k]
        sd["heavyball"] = {  # heavyball/utils.py:1527-1538
            "inner_group": dict(self.inner_group),  # a snapshot: the live dict keeps counting
            "use_ema": self.use_ema,
            "ema_decay": self.ema_decay,
            "compile_step": self.compile_step,
            "hessian_approx": self.hessian_approx,
            "precond_schedule": pickle.dumps(self.precond_schedule),
            "fallback_to_finite_differences": self.fallback_to_finite_differences,
            "_fallback_enabled": self._fallback_enabled,
            "hvp_interval": self.hvp_interval,
        }
        return sd

    def load_state_dict(self, state_dict):
        stats = state_dict.get("heavyball", {})
        for k, v in stats.items():  # heavyball/utils.py:1542-1549
            if k in ("stochastic_schedule", "precond_rng"):
                continue
            if k == "precond_schedule":
                v = _Unpickle(io.BytesIO(v)).load()
            if k == "inner_group":
                v = dict(v)  # not the caller's object: two optimizers loaded from one checkpoint must not share a counter
            setattr(self, k, v)
        sd = {k: v for k, v in state_dict.items() if k != "heavyball"}
        self._plans.clear()
        super().load_state_dict(sd)
        self._rehome_state()

    def _role_dtype(self, group, key: str) -> Optional[torch.dtype]:
        """Storage dtype of a loaded state tensor (heavyball/chainable.py:2452-2484 restores these after torch's cast)."""
        is_param_key = key == "param" or key.startswith("param::")
        mode = group.get("param_ecc") if is_param_key else group.get("ecc")
        if mode:
            prim, corr = _ECC_DTYPES[mode]
            return corr if key.endswith("::ecc") else prim
        return getattr(torch, group.get("storage_dtype", "float32"))

    def _rehome_state(self):
        """After ``load_state_dict`` the state tensors are fresh allocations in the parameter's dtype: cast them back to
        their storage dtype and move them into the slab, so that the kernels and ``optimizer.state`` share memory again."""
        for gi, group in enumerate(self.param_groups):
            if gi not in self._buckets:
                self._adopt_group(gi, group)
            for b in self._buckets[gi]:
                b.state_ready.clear()
                for i, p in enumerate(b.params):
                    if p not in self.state:
                        continue
                    for idx_state in self.state[p].values():
                        if not isinstance(idx_state, dict):
                            continue
                        for k in list(idx_state.keys()):
                            v = idx_state[k]
                            if not isinstance(v, torch.Tensor) or k == "step" or v.shape != p.shape:
                                continue
                            dt = self._role_dtype(group, k)
                            buf = b.slab.role(k, dt)
                            assert buf is not None
                            view = b.slab.view(k, i)
                            view.copy_(v.to(dt))
                            idx_state[k] = view
                    if group.get("param_ecc") and "param::ecc" not in self._state0(p):
                        self._state0(p)["param::ecc"] = b.slab.view("param::ecc", i)
                    if p.data.data_ptr() != b.slab.view("param", i).data_ptr():
                        view = b.slab.view("param", i)
                        view.copy_(p.data.to(view.dtype))
                        p.data = view


# ---------------------------------------------------------------------------------------------------------------
# AdamW / LaProp on the fused kernel
# ---------------------------------------------------------------------------------------------------------------
class _BucketPlan:
    """What one bucket's launch needs from step to step: the filled descriptor and the tables it points to."""

    __slots__ = ("bucket", "desc", "gdt", "params", "home", "keep", "device_index", "home_t", "ptrs_t", "ptrs_np")


class _StepPlan:
    """The launches of one parameter group as the general path last issued them, for ``FirstOrder._fast_step``."""

    __slots__ = ("sig", "buckets", "step_t", "state0", "n_state", "lr_t", "mars_key", "mars_w")


class FirstOrder(HBOptimizer):
    """AdamW-, LaProp-, ADOPT-, AdEMAMix- and NAdam-style optimizers: one call of ``hb_fused_step`` per parameter bucket."""

    _algo = _lib.ALGO_ADAM
    _fn_name = "update_by_adam"
    #: descriptor field -> state name, in the order the reference's guard lists them
    _moments = (("exp_avg", "exp_avg"), ("exp_avg_sq", "exp_avg_sq"))
    #: the index the reference's walk over the chain gives MARS' guard: behind the guards of the update transform
    _mars_idx = 2
    #: ``is_initialized`` entries of the update transform's guards
    _init_ids = frozenset({0})

    def _fn(self) -> str:
        fn = self._fn_name
        if self.update_clipping is not None:  # heavyball/chainable.py:2676-2684 swaps update_by_* for scale_by_*
            fn = fn.replace("update_by_", "scale_by_")
        return fn

    def _moment_keys(self, group) -> Dict[str, str]:
        """State-key names as the reference's index walk assigns them (heavyball/chainable.py:2347-2382): the guard that
        creates the moments is transform 0."""
        return {field: f"{self._fn()}_{name}_0" for field, name in self._moments}

    def _keys(self, group):
        mk = self._moment_keys(group)
        return mk["exp_avg"], mk["exp_avg_sq"], f"mars_mars_old_grad_{self._mars_idx}"

    def _state_fmt(self, group) -> Tuple[int, torch.dtype, Optional[torch.dtype]]:
        mode = group.get("ecc")
        if mode:
            prim, corr = _ECC_DTYPES[mode]
            return _lib.ECC_FMT[mode], prim, corr
        dt = getattr(torch, group.get("storage_dtype", "float32"))
        return _PLAIN_FMT[dt], dt, None

    def _ensure_state(self, group, b: Bucket, idx: List[int]):
        k_o = f"mars_mars_old_grad_{self._mars_idx}"
        _, prim, corr = self._state_fmt(group)
        mars = group.get("mars", False)
        names = list(self._moment_keys(group).values()) + ([k_o] if mars else [])
        ready = b.state_ready.setdefault((tuple(names), prim, corr), set())
        if len(ready) == len(b.params) or ready.issuperset(idx):
            # the caller may have dropped entries of optimizer.state since (all of them, or one parameter's): look at every one
            state, params, first = self.state, b.params, names[0]
            for i in idx:
                st = state.get(params[i])
                if st is None or first not in st.get(0, ()):
                    stale = set(ready)  # tensors whose slab ranges still hold the moments of the dropped entries
                    ready.clear()  # build the entries again
                    break
            else:
                return
        else:
            stale = ()
        for k in names:
            b.slab.role(k, prim)
            if corr is not None:
                b.slab.role(k + "::ecc", corr)
        init_ids = set(self._init_ids) | ({self._mars_idx} if mars else set())
        for i in idx:
            st = self._state0(b.params[i])
            if names[0] in st and (not mars or k_o in st):
                continue
            for k in names:
                fresh = k not in st
                st.setdefault(k, b.slab.view(k, i))
                if corr is not None:
                    st.setdefault(k + "::ecc", b.slab.view(k + "::ecc", i))
                if fresh and i in stale:  # a dropped entry starts from zero again, as the reference's zero_guard would
                    st[k].zero_()
                    if corr is not None:
                        st[k + "::ecc"].zero_()
            st.setdefault("is_initialized", set()).update(init_ids)
        ready.update(idx)

    def _step_scalars(self, group, step) -> dict:
        """The fp32 scalars of the step as the reference's 0-d tensors hold them (descriptor field -> python float)."""
        beta1, beta2 = self._betas(group, step)
        a1, oma1 = debiased_weights(beta1, step)
        a2, oma2 = debiased_weights(beta2, step)
        eps = float(f32(group["eps"])) if self._algo == _lib.ALGO_ADAM else float(f32(1e-8))  # chainable.py:868-881
        return dict(a1=a1, one_minus_a1=oma1, a2=a2, one_minus_a2=oma2, eps=eps)

    def _decay(self, group) -> Tuple[float, int]:
        """(the decay of ``p * (1 - decay * lr)``, extra descriptor flags)."""
        return group["weight_decay"], 0

    def _begin_step(self, group, work) -> bool:
        """Called once the active tensors are known.  Returns False when the step only warms a state up (no update)."""
        return True

    def _fill_bucket(self, d, b: Bucket, lst, group, step):
        """Per-bucket descriptor fields beyond the common ones; returns what must stay alive until the stream is done."""
        return None

    #: the step's scalars and descriptor are those of this class (no per-step hooks of a subclass): ``_fast_step`` may replay them
    _plannable = False

    def _plan_signature(self, group) -> tuple:
        """Everything, apart from the hyper-parameters that ``_fast_step`` reads afresh, that decides how a step is launched."""
        return (group["caution"], bool(group.get("mars", False)), bool(group.get("cautious_weight_decay", False)), group.get("ecc"),
                group.get("param_ecc"), group.get("storage_dtype"), self.rounding, self.promote, self.mars_write_grad,
                self.gradient_clipping, self.update_clipping, self._use_palm)  # fmt: skip

    def _fast_step(self, gi: int, group: dict) -> bool:
        """The step of a group whose every parameter has a gradient of the dtype, alignment and layout of the step before: the
        descriptors of that step are launched again with the new step number, scalars and gradient pointers.  Nothing is
        computed differently from the general path (tests/test_host_logic.py compares the scalars, the GPU tests the steps);
        anything out of the ordinary - a missing or differently typed gradient, a parameter whose data was rebound, emptied
        optimizer state, changed switches - returns False before anything was touched, and the general path takes the step."""
        plan = self._plans[gi]
        step_t = plan.step_t
        if (plan.sig != self._plan_signature(group) or group.get("_group_step") is not step_t or plan.state0.get("step") is not step_t
                or len(self.state) != plan.n_state):  # fmt: skip
            del self._plans[gi]
            return False
        base_lr = group["lr"]
        if type(base_lr) is not float:
            return False
        self._note_lr(group)
        staged = []
        helper = hostloop()
        for bp in plan.buckets:
            if helper is not None:  # the same checks in one C++ loop over the tensors
                if helper.collect(bp.params, bp.home_t, bp.ptrs_t, bp.gdt) != 0:
                    return False
                staged.append(None)
                continue
            grads = [p.grad for p in bp.params]
            try:
                ptrs = [g.data_ptr() for g in grads]
            except (AttributeError, RuntimeError):  # a parameter without a gradient, or a gradient without dense storage
                return False
            gdt = bp.gdt
            for g in grads:
                if g.dtype is not gdt or not g.is_contiguous():
                    return False
            low = 0
            for a in ptrs:
                low |= a
            if low & 15 or [p.data_ptr() for p in bp.params] != bp.home:
                return False
            staged.append(ptrs)
        n = step_t.item() + 1
        step_t.fill_(n)
        lr = step_lr_np(base_lr, n, group["warmup_steps"])
        group["prev_lr"] = plan.lr_t.fill_(float(lr))
        betas = group["betas"]
        beta1 = betas[0] if group.get("beta") is None else group["beta"]
        a1, oma1 = debiased_weights_np(beta1, n)
        a2, oma2 = debiased_weights_np(betas[1], n)
        eps = float(np.float32(group["eps"] if self._algo == _lib.ALGO_ADAM else 1e-8))
        omdl, neg_lr = float(_ONE32 - np.float32(group["weight_decay"]) * lr), float(-lr)
        if plan.sig[1]:
            key = (group["mars_gamma"], beta1)
            if plan.mars_key != key:
                plan.mars_key, plan.mars_w = key, mars_weights(group)
            mars_a, mars_oma = plan.mars_w
        else:
            mars_a, mars_oma = 0.0, 1.0
        L = _lib.lib()
        seed, step32 = self.rng_seed, n & 0xFFFFFFFF
        current = torch.cuda.current_device()
        for bp, ptrs in zip(plan.buckets, staged):
            b, d = bp.bucket, bp.desc
            table = b.grad_ptr_table(bp.gdt, ptrs) if ptrs is not None else b.grad_ptr_table_from((bp.gdt, bp.ptrs_np.tobytes()), bp.ptrs_t)
            d.grad_ptrs = table.data_ptr()
            d.a1, d.one_minus_a1, d.a2, d.one_minus_a2, d.eps = a1, oma1, a2, oma2, eps
            d.mars_a, d.one_minus_mars_a, d.neg_lr, d.one_minus_decay_lr = mars_a, mars_oma, neg_lr, omdl
            d.step, d.seed = step32, seed
            if bp.device_index == current:
                rc = L.hb_fused_step(d, current_stream_ptr(b.device))
            else:
                with torch.cuda.device(b.device):
                    rc = L.hb_fused_step(d, current_stream_ptr(b.device))
            _lib.check(rc, "hb_fused_step")
            self._last_launch = (d, (table, bp.keep))
        # The gradients go last: until the launches are queued nothing may free their memory, or an allocation made on the way
        # (a new pointer table) could be handed a gradient's block and be written ahead of the kernel that reads the gradient.
        if self.consume_grad:
            for bp in plan.buckets:
                if helper is not None:
                    helper.drop_grads(bp.params)
                    continue
                for p in bp.params:
                    p.grad = None
        return True

    #: take the un-fused form of the transform (scale_by_*, then update_param_) whenever a gradient is narrower than fp32: the
    #: reference's un-fused transform leaves its result in an update buffer of the gradient's dtype (MuonAdamW's vector route)
    _unfused_for_narrow_grads = False

    def _run_group(self, gi, group, active):
        self._run_gen(self._run_group_gen(gi, group, active))

    def _run_group_gen(self, gi, group, active):
        narrow = not self.promote and any(g.dtype != torch.float32 for _, g in active)
        unfused = self.update_clipping is not None or (self._unfused_for_narrow_grads and narrow)
        L = _lib.lib()
        step = group["step"]
        lr = f32(group["lr"])
        scal = self._step_scalars(group, step)
        if unfused and self._algo == _lib.ALGO_ADOPT:
            scal["eps"] = float(f32(1e-8))  # heavyball/chainable.py:1014-1023 passes no eps to utils.adopt: its default
        decay_py, decay_flags = self._decay(group)
        decay = f32(decay_py)
        omdl = float(1 - decay * lr)
        neg_lr = float(-lr)
        flags = 0
        mars = bool(group.get("mars", False))
        if mars:
            flags |= _lib.FLAG_MARS
            if self.mars_write_grad:
                flags |= _lib.FLAG_WRITE_GRAD
            mars_a, mars_oma = mars_weights(group)
        else:
            mars_a, mars_oma = 0.0, 1.0
        if group["caution"]:
            flags |= _lib.FLAG_CAUTION
        if group.get("cautious_weight_decay", False):
            flags |= _lib.FLAG_CAUTIOUS_WD
        flags |= decay_flags
        state_fmt, _, _ = self._state_fmt(group)
        moment_keys = self._moment_keys(group)
        k_o = f"mars_mars_old_grad_{self._mars_idx}"
        pecc = group.get("param_ecc")

        per_bucket: Dict[int, List] = {}
        for p, g in active:
            b, i = self._find_bucket(gi, p)
            per_bucket.setdefault(id(b), [b, []])[1].append((i, p, g))

        work = []  # (bucket, [(index, gradient)], gradient dtype)
        as_given = True  # every gradient went to the kernel as the caller handed it over (no cast, no copy)
        for b, items in per_bucket.values():
            if b.device.type != "cuda":
                raise _lib.HbError("the optimizer step runs on the GPU only: parameters must live on a CUDA/HIP device")
            self._check_home(b, items)
            self._ensure_state(group, b, [i for i, _, _ in items])
            by_dtype: Dict[torch.dtype, List] = {}
            f32_t, promote = torch.float32, self.promote
            for i, p, g in items:
                if g.is_sparse:
                    raise NotImplementedError("sparse gradients")
                dt = g.dtype
                if dt is not f32_t and (promote or dt not in _PLAIN_FMT):
                    g, dt, as_given = g.float(), f32_t, False
                if g.shape != p.shape:
                    raise ValueError(f"gradient shape {tuple(g.shape)} does not match parameter shape {tuple(p.shape)}")
                if g.data_ptr() & 15 or not g.is_contiguous() or g.device != b.device:
                    g, as_given = g.detach().to(b.device).clone(memory_format=torch.contiguous_format), False
                lst = by_dtype.get(dt)
                if lst is None:
                    lst = by_dtype[dt] = []
                lst.append((i, g))
            for gdt, lst in by_dtype.items():
                lst.sort(key=lambda t: t[0])
                work.append((b, lst, gdt))
        prologue = False
        if self.gradient_clipping is not None and mars:
            # heavyball/chainable.py:2694-2699: MARS, then the clip, then the transform.  The prologue runs as a pass of its
            # own (HB_FLAG_MARS_ONLY) that leaves the corrected gradients in the fp32 role "_clip"; the step proper then
            # runs without the MARS flag on the clipped slab
            for b, lst, gdt in work:
                self._mars_prologue(L, group, b, lst, gdt, step, mars_a, mars_oma, state_fmt, k_o)
            flags &= ~(_lib.FLAG_MARS | _lib.FLAG_WRITE_GRAD)
            mars = False
            prologue = True
            clipped = yield from self._clip_gradients_gen(L, group, work, step, gathered=True)
        elif self.gradient_clipping is not None:
            clipped = yield from self._clip_gradients_gen(L, group, work, step)
        else:
            clipped = [None] * len(work)
        plannable = (as_given and not unfused and self.gradient_clipping is None and not self._use_palm and self._plannable
                     and len(active) == len(group["params"]) and len(work) == len(per_bucket))
        plan_buckets = []
        if not self._begin_step(group, work):  # ADOPT's warm-up: only exp_avg_sq moves (and MARS' old gradient)
            flags = (flags & (_lib.FLAG_MARS | _lib.FLAG_WRITE_GRAD)) | _lib.FLAG_ADOPT_WARMUP
            scal = dict(scal, a2=1.0, one_minus_a2=0.0)
            unfused = False  # the warm-up skips the rest of the chain (WarmupGuard, heavyball/chainable.py:597-610)

        for (b, lst, gdt), clip in zip(work, clipped):
            offsets, numel = b.slab.meta()
            act = tuple(i for i, _ in lst)
            chunks, n_chunks = b.slab.chunks(act)
            d = _lib.HbStepDesc()
            d.param = b.slab.ptr("param")
            d.param_corr = b.slab.ptr("param::ecc")
            if clip is None:
                ptrs = [0] * len(b.params)
                for i, g in lst:
                    ptrs[i] = g.data_ptr()
                table = b.grad_ptr_table(gdt, ptrs)
                d.grad, d.grad_ptrs = None, table.data_ptr()
            else:
                table, gdt = clip[0], clip[1]  # the clipped gradients live in a slab role
                d.grad, d.grad_ptrs = table.data_ptr(), None
            for field, key in moment_keys.items():
                setattr(d, field, b.slab.ptr(key))
                setattr(d, field + "_corr", b.slab.ptr(key + "::ecc"))
            if mars:
                d.old_grad, d.old_grad_corr = b.slab.ptr(k_o), b.slab.ptr(k_o + "::ecc")
            d.offsets, d.numel, d.chunks = offsets.data_ptr(), numel.data_ptr(), chunks.data_ptr()
            d.caution_count = b.caution_scratch().data_ptr() if flags & _lib.FLAG_CAUTION else None
            d.n_chunks, d.n_tensors = n_chunks, len(b.params)
            d.algo, d.flags = self._algo, flags
            d.param_fmt = _lib.ECC_FMT[pecc] if pecc else _PLAIN_FMT[b.param_dtype]
            d.grad_fmt, d.state_fmt = _PLAIN_FMT[gdt], state_fmt
            for field, value in scal.items():
                setattr(d, field, value)
            d.mars_a, d.one_minus_mars_a = mars_a, mars_oma
            d.neg_lr, d.one_minus_decay_lr = neg_lr, omdl
            d.rng_mode, d.step, d.seed = self._rng_mode(), int(step) & 0xFFFFFFFF, self.rng_seed
            extra = self._fill_bucket(d, b, lst, group, step)
            if unfused:
                # heavyball/chainable.py:2676-2684: with update_clipping the chain is scale_by_* -> clip -> update_param_.
                # The step kernel only advances the moments and writes the update into the fp32 role "_update".
                b.slab.role("_update", torch.float32)
                d.update_out = b.slab.ptr("_update")
                d.flags = (flags & (_lib.FLAG_MARS | _lib.FLAG_WRITE_GRAD | _lib.FLAG_COUPLED_WD)) | _lib.FLAG_UPDATE_ONLY
                if mars and group["caution"]:
                    # the chain's tail compares the clipped update with the gradient as MARS left it (chainable.py:646 writes the
                    # corrected gradient into the gradient buffer): the step kernel has to write it there
                    d.flags |= _lib.FLAG_WRITE_GRAD
                d.caution_count = None
            with torch.cuda.device(b.device):
                rc = L.hb_fused_step(d, current_stream_ptr(b.device))
            _lib.check(rc, "hb_fused_step")
            self._last_launch = (d, (table, chunks, offsets, numel, clip, extra))  # kept for profiling harnesses
            if plannable:
                bp = _BucketPlan()
                bp.bucket, bp.desc, bp.gdt, bp.params, bp.home = b, d, gdt, b.params, b.home_ptrs()
                bp.keep, bp.device_index = (chunks, offsets, numel), b.device.index
                bp.home_t, bp.ptrs_t = torch.tensor(bp.home, dtype=torch.int64), torch.zeros(len(bp.home), dtype=torch.int64)
                bp.ptrs_np = bp.ptrs_t.numpy()
                plan_buckets.append(bp)
        if plannable:
            plan = _StepPlan()
            plan.sig, plan.buckets = self._plan_signature(group), plan_buckets
            plan.step_t, plan.state0, plan.n_state = group["_group_step"], self._state0(active[0][0]), len(self.state)
            plan.lr_t, plan.mars_key, plan.mars_w = torch.zeros((), dtype=torch.float32), None, None
            self._plans[gi] = plan
        if not unfused:
            return
        keep = None
        if self.update_clipping is not None:
            keep = yield (self.update_clipping, "_update", [(b, [i for i, _ in lst]) for b, lst, _ in work])
        decay_py = group["weight_decay"]  # update_param_ keeps decay a python float (heavyball/utils.py:2393-2406)
        for (b, lst, gdt), clip in zip(work, clipped):
            upd_role, upd_fmt = "_update", _lib.FMT_F32
            if gdt == torch.bfloat16:
                # the clip writes its result back into the bf16 update buffer through copy_stochastic_ (heavyball/utils.py:3231)
                wide, narrow = b.slab.role("_update", torch.float32), b.slab.role("_update16", torch.bfloat16)
                with torch.cuda.device(b.device):
                    _lib.check(L.hb_sr_bf16(wide.data_ptr(), narrow.data_ptr(), wide.numel(), self._rng_mode(), self.rng_seed,
                                            int(step) & 0xFFFFFFFF, _lib.STREAM_UPDATE_CLIP, 0, current_stream_ptr(b.device)), "hb_sr_bf16")  # fmt: skip
                upd_role, upd_fmt = "_update16", _lib.FMT_BF16
            elif gdt == torch.float16 and self.update_clipping is not None:
                # a float16 update buffer takes the clipped values through a plain cast (heavyball/utils.py:2363-2370 rounds
                # stochastically into bfloat16 only); the values stay in the fp32 role, every one of them a float16 number
                b.slab.role("_update", torch.float32)
                for i, _ in lst:  # this launch's tensors only: the bucket may hold tensors with gradients of another dtype
                    wide = b.slab.view("_update", i)
                    wide.copy_(wide.to(torch.float16))
            offsets, numel = b.slab.meta()
            chunks, n_chunks = b.slab.chunks(tuple(i for i, _ in lst))
            ptrs = [0] * len(b.params)
            for i, g in lst:
                ptrs[i] = g.data_ptr()
            table = b.grad_ptr_table(gdt, ptrs)  # caution compares the update with the gradient (MARS-corrected in place, if on)
            d = _lib.HbStepDesc()
            d.param, d.param_corr = b.slab.ptr("param"), b.slab.ptr("param::ecc")
            d.grad, d.grad_ptrs = None, table.data_ptr()
            if prologue:
                # MARS ran as a pass of its own and left the corrected gradients in a slab role instead of the caller's buffers
                # (heavyball/chainable.py:646 overwrites those); the clip that followed scaled them by a positive factor, which
                # keeps every sign bit, and the sign is all that caution reads
                d.grad, d.grad_ptrs, gdt = clip[0].data_ptr(), None, clip[1]
            d.exp_avg, d.state_fmt = b.slab.ptr(upd_role), upd_fmt
            d.offsets, d.numel, d.chunks = offsets.data_ptr(), numel.data_ptr(), chunks.data_ptr()
            d.caution_count = b.caution_scratch().data_ptr() if group["caution"] else None
            d.n_chunks, d.n_tensors = n_chunks, len(b.params)
            d.flags = flags & (_lib.FLAG_CAUTION | _lib.FLAG_CAUTIOUS_WD)
            d.param_fmt = _lib.ECC_FMT[pecc] if pecc else _PLAIN_FMT[b.param_dtype]
            d.grad_fmt = _PLAIN_FMT[gdt]
            d.neg_lr, d.one_minus_decay_lr = neg_lr, float(1 - decay_py * lr)
            d.rng_mode, d.step, d.seed = self._rng_mode(), int(step) & 0xFFFFFFFF, self.rng_seed
            with torch.cuda.device(b.device):
                _lib.check(L.hb_update_param(d, current_stream_ptr(b.device)), "hb_update_param")
            self._last_launch = (d, (table, chunks, offsets, numel, keep))


ShapeMap = dict


class AdamW(FirstOrder):
    """AdamW with HeavyBall's signature (heavyball/__init__.py:44-80), running ``update_by_adam`` on the fused kernel."""

    _algo = _lib.ALGO_ADAM
    _fn_name = "update_by_adam"
    _plannable = True

    def __init__(self, params, lr=0.0025, betas=(0.9, 0.99), eps=1e-8, weight_decay=0, cautious_weight_decay: bool = False,
                 warmup_steps=0, multi_tensor: bool = True, storage_dtype: str = "float32", mars: bool = False,
                 caution: bool = False, mars_gamma: float = 0.0025, gradient_clipping=use_default, update_clipping=use_default,
                 palm: bool = use_default, beta2_scale: float = 0.8, compile_step: bool = use_default, promote: bool = use_default,
                 ecc: Optional[str] = None, param_ecc: Optional[str] = None, orig_shapes: Optional[ShapeMap] = None, **kwargs):  # fmt: skip
        params, defaults = build_defaults(locals())
        super().__init__(params, defaults, gradient_clipping, update_clipping, palm)


class LaProp(FirstOrder):
    """LaProp with HeavyBall's signature (heavyball/__init__.py:740-776), running ``update_by_laprop`` on the fused kernel."""

    _algo = _lib.ALGO_LAPROP
    _fn_name = "update_by_laprop"
    _plannable = True

    def __init__(self, params, lr=0.0025, betas=(0.9, 0.99), eps=1e-8, weight_decay=0, cautious_weight_decay: bool = False,
                 warmup_steps=0, multi_tensor: bool = True, storage_dtype: str = "float32", mars: bool = False,
                 caution: bool = False, mars_gamma: float = 0.0025, gradient_clipping=use_default, update_clipping=use_default,
                 palm: bool = use_default, beta2_scale: float = 0.8, compile_step: bool = use_default, promote: bool = use_default,
                 ecc: Optional[str] = None, param_ecc: Optional[str] = None, orig_shapes: Optional[ShapeMap] = None, **kwargs):  # fmt: skip
        params, defaults = build_defaults(locals())
        super().__init__(params, defaults, gradient_clipping, update_clipping, palm)


class ADOPT(FirstOrder):
    """ADOPT with HeavyBall's signature (heavyball/__init__.py:640-681), running ``update_by_adopt`` on the fused kernel.

    The first step a tensor takes only sets ``exp_avg_sq = g*g`` (``_adopt_warmup_1`` under ``WarmupGuard``,
    heavyball/chainable.py:945-969, :587-610); as in the reference, a step in which *any* active tensor still lacks
    that warm-up is a warm-up step for all of them.  Afterwards the update divides by the second moment of the steps
    before and uses ``step - 1`` in the debiasing.
    """

    _algo = _lib.ALGO_ADOPT
    _fn_name = "update_by_adopt"
    _mars_idx = 3  # ZeroGuard 0, WarmupGuard 1, the transform itself 2

    def __init__(self, params, lr=0.0025, betas=(0.9, 0.99), eps=1e-8, weight_decay=0, cautious_weight_decay: bool = False,
                 warmup_steps=0, multi_tensor: bool = True, storage_dtype: str = "float32", mars: bool = False,
                 caution: bool = False, mars_gamma: float = 0.0025, gradient_clipping=use_default, update_clipping=use_default,
                 palm: bool = use_default, beta2_scale: float = 0.8, compile_step: bool = use_default, promote: bool = use_default,
                 ecc: Optional[str] = None, param_ecc: Optional[str] = None, orig_shapes: Optional[ShapeMap] = None, **kwargs):  # fmt: skip
        params, defaults = build_defaults(locals())
        super().__init__(params, defaults, gradient_clipping, update_clipping, palm)

    def _step_scalars(self, group, step) -> dict:
        beta1, beta2 = self._betas(group, step)
        before = step - 1  # heavyball/chainable.py:961
        a1, oma1 = debiased_weights(beta1, before) if int(before) > 0 else (1.0, 0.0)
        a2, oma2 = debiased_weights(beta2, before + 1)  # heavyball/utils.py:2303-2304
        return dict(a1=a1, one_minus_a1=oma1, a2=a2, one_minus_a2=oma2, eps=float(f32(group["eps"])))

    def _begin_step(self, group, work) -> bool:
        states = [self._state0(b.params[i]) for b, lst, _ in work for i, _ in lst]
        if min(st.get("_warmup_1", 0) for st in states) < 1:
            for st in states:
                st["_warmup_1"] = st.get("_warmup_1", 0) + 1
            return False
        for st in states:
            st.setdefault("is_initialized", set()).add(1)
        return True


class AdEMAMix(FirstOrder):
    """AdEMAMix with HeavyBall's signature (heavyball/__init__.py:124-164), running ``update_by_ademamix`` on the fused kernel:
    a fast and a slow momentum, ``update = (fast + alpha * slow) / denom``, with the warm-up schedules of alpha and of
    beta3's half-life (heavyball/utils.py:290-334)."""

    _algo = _lib.ALGO_ADEMAMIX
    _fn_name = "update_by_ademamix"
    _moments = (("exp_avg", "exp_avg_fast"), ("exp_avg_slow", "exp_avg_slow"), ("exp_avg_sq", "exp_avg_sq"))

    def __init__(self, params, lr=0.001, betas=(0.9, 0.999, 0.9999), eps=1e-8, weight_decay=0, cautious_weight_decay: bool = False,
                 alpha: float = 2.0, beta3_warmup: Optional[int] = None, alpha_warmup: Optional[int] = None, warmup_steps=0,
                 multi_tensor: bool = True, storage_dtype: str = "float32", mars: bool = False, caution: bool = False,
                 mars_gamma: float = 0.0025, gradient_clipping=use_default, update_clipping=use_default,
                 compile_step: bool = use_default, promote: bool = use_default, ecc: Optional[str] = None,
                 param_ecc: Optional[str] = None, orig_shapes: Optional[ShapeMap] = None, **kwargs):  # fmt: skip
        if len(betas) != 3:
            raise ValueError("AdEMAMix expects betas with three coefficients.")
        params, defaults = build_defaults(locals())
        super().__init__(params, defaults, gradient_clipping, update_clipping)

    @staticmethod
    def _alpha_at(step: int, alpha_end: float, warmup) -> float:
        """heavyball/utils.py:290-298 with alpha_start = 0."""
        if warmup is None or warmup <= 0 or step >= warmup:
            return alpha_end
        a = step / float(warmup)
        return (1.0 - a) * 0.0 + a * alpha_end

    @staticmethod
    def _beta3_at(step: int, beta_end: float, beta_start: float, warmup, eps: float = 1e-8) -> float:
        """heavyball/utils.py:301-318: linear in the half-life ``log(0.5) / log(beta) - 1``, not in beta."""
        if warmup is None or warmup <= 0 or step >= warmup:
            return beta_end
        a = step / float(warmup)
        hl0 = math.log(0.5) / math.log(beta_start + eps) - 1
        hl1 = math.log(0.5) / math.log(beta_end + eps) - 1
        beta = math.pow(0.5, 1.0 / ((1.0 - a) * hl0 + a * hl1 + 1.0))
        return min(max(beta, 0.0), 1.0 - eps)

    def _step_scalars(self, group, step) -> dict:
        betas = group["betas"]
        if len(betas) != 3:
            raise ValueError("AdEMAMix expects betas=(beta1, beta2, beta3).")
        beta1, beta2, beta3_final = betas
        s = int(step)
        alpha = self._alpha_at(s, group["alpha"], group.get("alpha_warmup"))
        beta3 = self._beta3_at(s, beta3_final, beta1, group.get("beta3_warmup"))
        a1, oma1 = debiased_weights(f32(beta1), step)
        a2, oma2 = debiased_weights(f32(beta2), step)
        a3, oma3 = lerp_weights(f32(beta3))  # the slow momentum is not debiased (heavyball/utils.py:2105)
        return dict(a1=a1, one_minus_a1=oma1, a2=a2, one_minus_a2=oma2, a3=a3, one_minus_a3=oma3, alpha=float(f32(alpha)),
                    eps=float(f32(group["eps"])))  # fmt: skip


class NAdam(FirstOrder):
    """NAdam with HeavyBall's signature (heavyball/__init__.py:83-121), running ``update_by_nadam`` on the fused kernel.

    Per tensor the reference keeps the running product of the momentum schedule, ``mu_product`` (a 0-d tensor in the
    storage dtype, heavyball/chainable.py:272-274), and derives two weights from it each step
    (heavyball/utils.py:398-409).  Those are host-known scalars: the host advances a CPU copy of the products with the
    same torch ops, uploads them (they stay visible as ``optimizer.state[p][0]["update_by_nadam_mu_product_1"]``) and
    hands the kernel two weights per tensor.  Weight decay that is not decoupled enters through the gradient and is
    taken out of the finished update (heavyball/utils.py:350-379).
    """

    _algo = _lib.ALGO_NADAM
    _fn_name = "update_by_nadam"
    _mars_idx = 3  # ZeroGuard 0, GeneralGuard 1 (mu_product), the transform itself 2
    _init_ids = frozenset({0, 1})

    @property
    def MU_KEY(self) -> str:
        return f"{self._fn()}_mu_product_1"  # scale_by_nadam_... under update_clipping

    def __init__(self, params, lr=0.002, betas=(0.9, 0.999), eps=1e-8, weight_decay=0, cautious_weight_decay: bool = False,
                 momentum_decay: float = 4e-3, decoupled_weight_decay: bool = False, warmup_steps=0, multi_tensor: bool = True,
                 storage_dtype: str = "float32", mars: bool = False, caution: bool = False, mars_gamma: float = 0.0025,
                 gradient_clipping=use_default, update_clipping=use_default, palm: bool = use_default, beta2_scale: float = 0.8,
                 compile_step: bool = use_default, promote: bool = use_default, ecc: Optional[str] = None,
                 param_ecc: Optional[str] = None, orig_shapes: Optional[ShapeMap] = None, **kwargs):  # fmt: skip
        params, defaults = build_defaults(locals())
        super().__init__(params, defaults, gradient_clipping, update_clipping, palm)

    def _step_scalars(self, group, step) -> dict:
        beta1, beta2 = self._betas(group, step)
        a1, oma1 = lerp_weights(beta1)  # heavyball/utils.py:394: beta1 as it is
        a2, oma2 = debiased_weights(beta2, step)
        return dict(a1=a1, one_minus_a1=oma1, a2=a2, one_minus_a2=oma2, eps=float(f32(group["eps"])),
                    coupled_wd=float(f32(float(group["weight_decay"]))))  # fmt: skip

    def _decay(self, group) -> Tuple[float, int]:
        wd = float(group["weight_decay"])
        if wd == 0:
            return 0.0, 0
        if group.get("decoupled_weight_decay", False):
            return wd, 0
        return 0.0, _lib.FLAG_COUPLED_WD

    def _mu_host(self, group, b: Bucket) -> torch.Tensor:
        """CPU copy of the bucket's mu_product values, [n_tensors] in the storage dtype; ones until a tensor first steps."""
        host = getattr(b, "mu_host", None)
        if host is None:
            dt = getattr(torch, group.get("storage_dtype", "float32"))
            host = b.mu_host = torch.ones(len(b.params), dtype=dt)
            b.mu_dev = torch.ones(len(b.params), dtype=dt, device=b.device)
        return host

    def _fill_bucket(self, d, b: Bucket, lst, group, step):
        beta1, _ = self._betas(group, step)
        md = torch.as_tensor(group["momentum_decay"], dtype=torch.float32)  # heavyball/utils.py:341-347
        base = torch.tensor(0.96, dtype=torch.float32)
        step_f = step.to(torch.float32)
        mu = beta1 * (1 - 0.5 * torch.pow(base, step_f * md))
        mu_next = beta1 * (1 - 0.5 * torch.pow(base, (step_f + 1) * md))
        host = self._mu_host(group, b)
        act = torch.tensor([i for i, _ in lst], dtype=torch.int64)
        host[act] = (host[act].to(torch.float32) * mu).to(host.dtype)  # heavyball/utils.py:398-399: mp_.mul_(mu), stored in the storage dtype
        mp32 = host.to(torch.float32)
        one = torch.ones((), dtype=torch.float32)
        weights = torch.stack([(one - mu) / (one - mp32), mu_next / (one - mp32 * mu_next)], dim=1).contiguous()  # :403-408
        stage_w, stage_m = weights.pin_memory(), host.clone().pin_memory()
        dev_w = stage_w.to(b.device, non_blocking=True)
        b.mu_dev.copy_(stage_m, non_blocking=True)
        for i, _ in lst:
            self._state0(b.params[i]).setdefault(self.MU_KEY, b.mu_dev[i])
        d.tensor_scalars = dev_w.data_ptr()
        return dev_w, stage_w, stage_m

    def _rehome_state(self):
        super()._rehome_state()
        for gi, group in enumerate(self.param_groups):
            for b in self._buckets.get(gi, []):
                loaded = [(i, self.state[p][0][self.MU_KEY]) for i, p in enumerate(b.params)
                          if p in self.state and isinstance(self.state[p].get(0), dict) and self.MU_KEY in self.state[p][0]]  # fmt: skip
                if not loaded:
                    continue
                host = self._mu_host(group, b)
                for i, v in loaded:
                    host[i] = v.detach().to("cpu", host.dtype)
                b.mu_dev.copy_(host)
                for i, _ in loaded:
                    self.state[b.params[i]][0][self.MU_KEY] = b.mu_dev[i]

"""Muon (heavyball/__init__.py:684-737) on the HIP kernels: Nesterov-EMA momentum, Newton-Schulz orthogonalisation of
every parameter with two or more dimensions, then the plain parameter update."""

import ctypes
from typing import Dict, List, Optional

import torch

from . import _lib
from .optim import FirstOrder, HBOptimizer, _ECC_DTYPES, _PLAIN_FMT, beta_debias, build_defaults, current_stream_ptr, f32, lerp_weights, mars_weights, use_default

_NS_UPDATE_FLAG = {torch.float32: 0, torch.bfloat16: _lib.NS_BF16_UPDATE, torch.float16: _lib.NS_F16_UPDATE}
#: per-iteration (a, b, c) of zeropower_via_newtonschulz5 (heavyball/utils.py:561-567)
NS_COEFFS = (
    (4.0848, -6.8946, 2.9270),
    (3.9505, -6.3029, 2.6377),
    (3.7418, -5.5913, 2.3037),
    (2.8769, -3.1427, 1.2046),
    (2.8366, -3.0525, 1.2012),
)
#: legacy_zeropower_via_newtonschulz5 (heavyball/utils.py:639)
LEGACY_COEFFS = ((3.4445, -4.7750, 2.0315),) * 5

#: msign(x, 10) (heavyball/utils.py:587-602, :619): the polynomials of arXiv 2505.16932v3, all but the last divided by a safety
#: factor (a / 1.01, b / 1.01^3, c / 1.01^5), the last one repeated to fill the ten steps
_POLAR = (
    (8.28721201814563, -23.595886519098837, 17.300387312530933),
    (4.107059111542203, -2.9478499167379106, 0.5448431082926601),
    (3.9486908534822946, -2.908902115962949, 0.5518191394370137),
    (3.3184196573706015, -2.488488024314874, 0.51004894012372),
    (2.300652019954817, -1.6689039845747493, 0.4188073119525673),
    (1.891301407787398, -1.2679958271945868, 0.37680408948524835),
    (1.8750014808534479, -1.2500016453999487, 0.3750001645474248),
)
POLAR_COEFFS = tuple((a / 1.01, b / 1.01**3, c / 1.01**5) for a, b, c in _POLAR) + ((1.875, -1.25, 0.375),) * 3

#: module-level switch of the reference (heavyball/utils.py:25): "newtonschulz", "legacy_newtonschulz" or "thinky_polar_express"
zeroth_power_mode = "newtonschulz"


def ns_coefficients(coeffs) -> List[float]:
    """The three floats per iteration that ``hb_ns5`` and its relatives take, with the reference's CPU rounding of the scalars.

    ``y = c * s`` multiplies the bf16 matrix by the scalar at fp32 precision, but ``y.diagonal().add_(b)`` is an in-place
    bf16 op whose scalar operand is first cast to the tensor's dtype (heavyball/utils.py:569-572 as executed by ATen on
    CPU): ``a`` and ``b`` therefore enter as their bf16 roundings, ``c`` as an fp32 value.
    """
    out = []
    for a, b, c in coeffs:
        out += [float(torch.tensor(a).bfloat16()), float(torch.tensor(b).bfloat16()), float(f32(c))]
    return out


class Muon(HBOptimizer):
    """Muon with HeavyBall's signature (heavyball/__init__.py:684-737).

    Chain of the reference: a momentum transform -> ``orthogonalize_update`` (heavyball/chainable.py:1117-1126) ->
    ``update_param_`` (heavyball/utils.py:2393-2406).  The momentum is ``nesterov_ema`` by default (:1135-1138);
    ``nesterov=False`` selects ``exp_avg`` (:652-653), ``heavyball_momentum=True`` selects ``heavyball_momentum`` or, with
    ``nesterov``, ``nesterov_momentum`` (heavyball/__init__.py:723-729).  Parameters with fewer than two dimensions skip the
    orthogonalisation and are updated with the momentum direction itself, as in the reference.
    """

    def __init__(self, params, lr=0.0025, betas=(0.9, 0.99), eps=1e-8, weight_decay=0, cautious_weight_decay: bool = False,
                 warmup_steps=0, multi_tensor: bool = True, storage_dtype: str = "float32", mars: bool = False,
                 caution: bool = False, mars_gamma: float = 0.0025, gradient_clipping=use_default, update_clipping=use_default,
                 palm: bool = use_default, beta2_scale: float = 0.8, nesterov: bool = True, heavyball_momentum: bool = False,
                 compile_step: bool = use_default, promote: bool = use_default, ecc: Optional[str] = None,
                 param_ecc: Optional[str] = None, orig_shapes=None, **kwargs):  # fmt: skip
        params, defaults = build_defaults(locals())
        # heavyball/__init__.py:723-729: which momentum transform heads the chain; the state is named after it
        if heavyball_momentum:
            self._mom_mode = _lib.MOM_NESTEROV_HEAVYBALL if nesterov else _lib.MOM_HEAVYBALL
            self.KEY = "nesterov_momentum_momentum_2" if nesterov else "heavyball_momentum_momentum_2"
        elif not nesterov:
            self._mom_mode = _lib.MOM_EMA
            self.KEY = "exp_avg_exp_avg_2"
        super().__init__(params, defaults, gradient_clipping, update_clipping, palm)
        self._workspace: Dict[torch.device, torch.Tensor] = {}

    KEY = "nesterov_ema_momentum_2"  # heavyball/chainable.py:2347-2382: update_param's walk gives the momentum guard index 2

    @property
    def _mars_idx(self) -> int:
        """MARS' guard sits two places behind the momentum's in that walk (mars_mars_old_grad_4; _6 for MuonAdamW)."""
        return int(self.KEY.rsplit("_", 1)[1]) + 2

    _mom_mode = _lib.MOM_NESTEROV_EMA
    INIT = frozenset({0, 1, 2})

    def _ws(self, device, nbytes: int) -> torch.Tensor:
        ws = self._workspace.get(device)
        if ws is None or ws.numel() < nbytes:
            ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
            self._workspace[device] = ws
        return ws

    def _scratch64(self, device, key, n: int) -> torch.Tensor:
        """A float64 device buffer of at least ``n`` elements that lives as long as the optimizer, one per ``key``."""
        pool = self.__dict__.setdefault("_scratch64_pool", {})
        buf = pool.get(key)
        if buf is None or buf.numel() < n or buf.device != device:
            buf = pool[key] = torch.empty(max(n, 1), dtype=torch.float64, device=device)
        return buf

    #: upper bound on the Newton-Schulz scratch of one grouped call; a bucket whose matrices need more is split
    ns_workspace_limit = 16 << 30
    #: let the last Newton-Schulz product apply the step to fp32 parameters itself where the chain allows it (same arithmetic as
    #: hb_update_param; False keeps the two launches apart, which tests use to compare the two routes)
    fuse_update_into_newton_schulz = True

    def _ns_parts(self, L, mats):
        """Splits ``[(index, rows, cols), ...]`` into runs whose scratch stays under ``ns_workspace_limit``."""
        parts, cur, cur_bytes = [], [], 0
        for m in mats:
            r, c, nb = ctypes.c_int64(m[1]), ctypes.c_int64(m[2]), ctypes.c_int64()
            _lib.check(L.hb_ns5_batched_workspace_bytes(1, ctypes.byref(r), ctypes.byref(c), ctypes.byref(nb)))
            need = nb.value
            if cur and cur_bytes + need > self.ns_workspace_limit:
                parts.append(cur)
                cur, cur_bytes = [], 0
            cur.append(m)
            cur_bytes += need
        if cur:
            parts.append(cur)
        return parts

    def _run_group(self, gi, group, active):
        self._run_gen(self._run_group_gen(gi, group, active))

    def _run_group_gen(self, gi, group, active):
        active = [(p, g) for p, g in active if p.numel() > 0]  # an empty tensor has nothing to orthogonalise or update
        if not active:
            return
        L = _lib.lib()
        step = group["step"]
        lr = f32(group["lr"])
        raw_beta = group["betas"][0] if group.get("beta") is None else group["beta"]
        if self._mom_mode == _lib.MOM_NESTEROV_EMA:
            a = 1 - f32(raw_beta)  # _lerp(state, grad, beta) with the raw beta (heavyball/utils.py:768, :1847)
            a_f, oma_f = float(a), float(1 - a)
        elif self._mom_mode == _lib.MOM_EMA:
            a_f, oma_f = lerp_weights(f32(beta_debias(raw_beta, step)))  # heavyball/chainable.py:653: python beta, int64 step
        else:
            a_f, oma_f = float(f32(raw_beta)), 0.0  # heavyball/utils.py:737-749 multiply by beta itself
        decay = group["weight_decay"]
        omdl = float(1 - decay * lr)  # update_param_ keeps decay a python float (heavyball/utils.py:2389, :2393-2406)
        neg_lr = float(-lr)
        mode = zeroth_power_mode
        flags = 0
        if group["caution"]:
            flags |= _lib.FLAG_CAUTION
        if group.get("cautious_weight_decay", False):
            flags |= _lib.FLAG_CAUTIOUS_WD
        pecc = group.get("param_ecc")
        # storage of the momentum (zero_guard with the group's ecc / storage_dtype, heavyball/chainable.py:277-301)
        if group.get("ecc"):
            mom_prim, mom_corr = _ECC_DTYPES[group["ecc"]]
            mom_fmt = _lib.ECC_FMT[group["ecc"]]
        else:
            mom_prim, mom_corr = getattr(torch, group.get("storage_dtype", "float32")), None
            mom_fmt = _PLAIN_FMT[mom_prim]

        mars = bool(group.get("mars"))
        k_o = f"mars_mars_old_grad_{self._mars_idx}"
        init_ids = set(self.INIT) | ({self._mars_idx} if mars else set())
        if mars:
            mars_a, mars_oma = mars_weights(group)

        per_bucket: Dict[int, List] = {}
        for p, g in active:
            b, i = self._find_bucket(gi, p)
            per_bucket.setdefault(id(b), [b, []])[1].append((i, p, g))
        prepared = []
        for b, items in per_bucket.values():
            if b.device.type != "cuda":
                raise _lib.HbError("the optimizer step runs on the GPU only: parameters must live on a CUDA/HIP device")
            self._check_home(b, items)
            b.slab.role(self.KEY, mom_prim)
            if mom_corr is not None:
                b.slab.role(self.KEY + "::ecc", mom_corr)
            b.slab.role("_update", torch.float32)
            if mars:  # stored like the momentum (zero_guard with the same group settings)
                b.slab.role(k_o, mom_prim)
                if mom_corr is not None:
                    b.slab.role(k_o + "::ecc", mom_corr)
            by_dtype: Dict[torch.dtype, List] = {}
            for i, p, g in items:
                st = self._state0(p)
                for key in (self.KEY, k_o) if mars else (self.KEY,):
                    if key not in st:
                        st[key] = b.slab.view(key, i)
                        if mom_corr is not None:
                            st[key + "::ecc"] = b.slab.view(key + "::ecc", i)
                        st.setdefault("is_initialized", set()).update(init_ids)
                if self.promote and g.dtype != torch.float32:
                    g = g.float()
                if g.dtype not in _PLAIN_FMT:
                    g = g.float()
                if not g.is_contiguous() or g.data_ptr() % 16 or g.device != b.device:
                    g = g.to(b.device).clone(memory_format=torch.contiguous_format)
                by_dtype.setdefault(g.dtype, []).append((i, g))
            for lst in by_dtype.values():
                lst.sort(key=lambda t: t[0])
            prepared.append((b, items, by_dtype))
        # gradient_clipping (heavyball/chainable.py:2696-2699) acts on the update before the momentum transform
        clipped = {}
        if self.gradient_clipping is not None or mars:
            work = [(b, lst, gdt) for b, _, by_dtype in prepared for gdt, lst in by_dtype.items()]
            # MARS heads the chain (heavyball/chainable.py:2698-2699, :642-647): a pass of its own leaves the corrected gradients,
            # rounded to the gradient dtype, in the fp32 role "_clip"; clipping and the momentum go on from there
            for b, lst, gdt in work if mars else ():
                self._mars_prologue(L, group, b, lst, gdt, step, mars_a, mars_oma, mom_fmt, k_o)
            for (b, _, gdt), res in zip(work, (yield from self._clip_gradients_gen(L, group, work, step, gathered=mars))):
                clipped[(id(b), gdt)] = res
        keep = []
        stepped = set()  # (bucket, tensor) whose parameter the last Newton-Schulz product has already updated
        sumsq = {}  # (bucket, tensor) -> (address, count) of the partial sums of squares the momentum kernel left for it
        tables = {}  # (bucket, gradient dtype) -> device table of gradient pointers
        for b, items, by_dtype in prepared:
            offsets, numel = b.slab.meta()
            stream = current_stream_ptr(b.device)
            with torch.cuda.device(b.device):
                for gdt, lst in by_dtype.items():
                    act = tuple(i for i, _ in lst)
                    chunks, n_chunks = b.slab.chunks(act)
                    clip = clipped.get((id(b), gdt))
                    ptrs = [0] * len(b.params)
                    for i, g in lst:
                        ptrs[i] = g.data_ptr()
                    table = tables[(id(b), gdt)] = b.grad_ptr_table(gdt, ptrs)  # the raw gradients: caution compares the update against them
                    if clip is None:
                        g_slab, g_table, g_fmt = None, table.data_ptr(), _PLAIN_FMT[gdt]
                    else:  # the clipped gradients live in a slab role
                        g_slab, g_table, g_fmt = clip[0].data_ptr(), None, _PLAIN_FMT[clip[1]]
                    keep.append((table, chunks, lst, clip))
                    # the momentum kernel leaves the sums of squares of the update it writes, a few doubles per chunk, so that
                    # Newton-Schulz' norm needs no pass of its own over the update
                    per_chunk = L.hb_momentum_sumsq_parts_per_chunk()
                    parts = self._scratch64(b.device, ("sumsq", id(b), gdt), n_chunks * per_chunk)
                    first = 0
                    for i in act:
                        count = -(-b.slab.numels[i] // _lib.chunk_elems())
                        sumsq[(id(b), i)] = (parts.data_ptr() + 8 * first * per_chunk, count * per_chunk)
                        first += count
                    _lib.check(L.hb_momentum_sumsq(b.slab.ptr(self.KEY), b.slab.ptr(self.KEY + "::ecc"), mom_fmt, b.slab.ptr("_update"), g_slab,
                                                   g_table, g_fmt, offsets.data_ptr(), numel.data_ptr(), chunks.data_ptr(), n_chunks,
                                                   self._mom_mode, a_f, oma_f, self._rng_mode(), self.rng_seed, int(step) & 0xFFFFFFFF,
                                                   parts.data_ptr(), stream), "hb_momentum_sumsq")  # fmt: skip
                # orthogonalise every update with two or more dimensions (heavyball/chainable.py:1117-1126)
                if mode not in ("newtonschulz", "legacy_newtonschulz", "thinky_polar_express"):
                    # "qr", "svd", "legacy_svd" (heavyball/utils.py:798-806) are factorisations, not this iteration
                    raise NotImplementedError(f"zeroth_power_mode={mode!r}")
                # every matrix of the bucket goes through Newton-Schulz in the same grouped launches; under the legacy mode the
                # square ones take the legacy coefficient table and input rounding (heavyball/utils.py:790-795), under
                # "thinky_polar_express" the ten-step schedule of msign (:796-797, in a call of their own), the others the default
                # with 16-bit gradients the reference's update buffer has their dtype and Newton-Schulz normalises it there
                # (per matrix: a bucket may hold gradients of several dtypes)
                ns_flags = {i: _NS_UPDATE_FLAG[gdt] for gdt, lst in by_dtype.items() for i, _ in lst}
                # an fp32 parameter that nothing else looks at between Newton-Schulz and update_param_ (no caution, whose mask needs
                # the finished update of the whole tensor, and no clip of the update) takes its step in the epilogue of the last
                # product: the update is never written out and read back.  Matrices of the 128-wide kernel only: the 256-wide one
                # runs a single workgroup per compute unit, and the longer epilogue costs more there than the pass it saves.
                fuse_tail = (self.fuse_update_into_newton_schulz and not group["caution"] and self.update_clipping is None and not pecc
                             and b.param_dtype == torch.float32)  # fmt: skip
                tail_flags = (_lib.NS_APPLY_TO_PARAM | (_lib.NS_CAUTIOUS_WD if flags & _lib.FLAG_CAUTIOUS_WD else 0)) if fuse_tail else 0
                param_step = (ctypes.c_float * 2)(omdl, neg_lr)
                fused = {i for i, r, c in ((i, p.shape[0], p.numel() // p.shape[0]) for i, p, _ in items if p.dim() >= 2)
                         if fuse_tail and L.hb_ns_tile(r, c) == 128}  # fmt: skip
                mats = []
                for i, p, _ in items:
                    if p.dim() < 2:
                        continue
                    rows, cols = p.shape[0], p.numel() // p.shape[0]
                    mats.append((i, rows, cols))
                coeff_tables = {False: ns_coefficients(NS_COEFFS), True: ns_coefficients(LEGACY_COEFFS), "polar": ns_coefficients(POLAR_COEFFS)}
                polar = [m for m in mats if mode == "thinky_polar_express" and m[1] == m[2]]
                plain = [m for m in mats if not (mode == "thinky_polar_express" and m[1] == m[2])]
                for part, n_steps in [(q, 5) for q in self._ns_parts(L, plain)] + [(q, 10) for q in self._ns_parts(L, polar)]:
                    n = len(part)
                    legacy = [mode == "legacy_newtonschulz" and r == c for _, r, c in part]
                    rows_a = (ctypes.c_int64 * n)(*[r for _, r, _ in part])
                    cols_a = (ctypes.c_int64 * n)(*[c for _, _, c in part])
                    ptrs = (ctypes.c_void_p * n)(*[b.slab.view("_update", i).data_ptr() for i, _, _ in part])
                    outs = (ctypes.c_void_p * n)(*[b.slab.view("param" if i in fused else "_update", i).data_ptr() for i, _, _ in part])
                    scale = (ctypes.c_float * n)(*[max(1, r / c) ** 0.5 for _, r, c in part])  # heavyball/utils.py:808-809
                    base = (ctypes.c_int64 * n)(*[int(b.slab.offsets_np[i]) for i, _, _ in part])
                    arr = (ctypes.c_float * (3 * n_steps * n))(*[x for lg in legacy for x in coeff_tables["polar" if n_steps == 10 else lg]])
                    flag_a = (ctypes.c_int32 * n)(*[ns_flags[i] | int(lg) | (tail_flags if i in fused else 0)
                                                    for (i, _, _), lg in zip(part, legacy)])  # fmt: skip
                    ss_ptr = (ctypes.c_void_p * n)(*[sumsq[(id(b), i)][0] for i, _, _ in part])
                    ss_cnt = (ctypes.c_int32 * n)(*[sumsq[(id(b), i)][1] for i, _, _ in part])
                    nbytes = ctypes.c_int64()
                    _lib.check(L.hb_ns5_batched_workspace_bytes(n, rows_a, cols_a, ctypes.byref(nbytes)))
                    ws = self._ws(b.device, nbytes.value)
                    _lib.check(L.hb_ns_batched_steps(n, ptrs, outs, rows_a, cols_a, n_steps, arr, flag_a, 1e-7, scale, param_step, ss_ptr,
                                                     ss_cnt, self._rng_mode(), self.rng_seed, int(step) & 0xFFFFFFFF, base,
                                                     ws.data_ptr(), ws.numel(), stream), "hb_ns_batched_steps")  # fmt: skip
                stepped.update((id(b), i) for i in fused)
        if self.update_clipping is not None:  # heavyball/chainable.py:2700-2701: on the finished update of the whole group
            keep.append((yield (self.update_clipping, "_update", [(b, sorted(i for i, _, _ in items)) for b, items, _ in prepared])))
            for b, items, by_dtype in prepared:
                if torch.bfloat16 in by_dtype:
                    # the clip writes its result back into the bf16 update buffer through copy_stochastic_ (heavyball/utils.py:3231)
                    wide, narrow = b.slab.role("_update", torch.float32), b.slab.role("_update16", torch.bfloat16)
                    with torch.cuda.device(b.device):
                        _lib.check(L.hb_sr_bf16(wide.data_ptr(), narrow.data_ptr(), wide.numel(), self._rng_mode(), self.rng_seed,
                                                int(step) & 0xFFFFFFFF, _lib.STREAM_UPDATE_CLIP, 0, current_stream_ptr(b.device)), "hb_sr_bf16")  # fmt: skip
                # a float16 update buffer takes the clipped values through a plain cast (heavyball/utils.py:2348-2349); they stay in
                # the fp32 role, every one of them a float16 number
                for i, _ in by_dtype.get(torch.float16, ()):
                    wide = b.slab.view("_update", i)
                    wide.copy_(wide.to(torch.float16))
        for b, items, by_dtype in prepared:
            offsets, numel = b.slab.meta()
            stream = current_stream_ptr(b.device)
            with torch.cuda.device(b.device):
                # p <- p * (1 - decay * lr) + update * (-lr) for everything (heavyball/utils.py:2373-2406)
                for gdt, lst in by_dtype.items():
                    act = tuple(i for i, _ in lst if (id(b), i) not in stepped)  # the others took their step inside Newton-Schulz
                    if not act:
                        continue
                    chunks, n_chunks = b.slab.chunks(act)
                    table = tables[(id(b), gdt)]
                    d = _lib.HbStepDesc()
                    d.param, d.param_corr = b.slab.ptr("param"), b.slab.ptr("param::ecc")
                    d.grad, d.grad_ptrs, d.grad_fmt = None, table.data_ptr(), _PLAIN_FMT[gdt]
                    if mars:
                        # caution compares the update with the gradient as MARS left it; a clip after MARS scales that by a
                        # positive factor, which keeps every sign
                        d.grad, d.grad_ptrs, d.grad_fmt = b.slab.ptr("_clip"), None, _lib.FMT_F32
                    d.exp_avg = b.slab.ptr("_update")
                    if self.update_clipping is not None and gdt == torch.bfloat16:
                        d.exp_avg, d.state_fmt = b.slab.ptr("_update16"), _lib.FMT_BF16
                    d.offsets, d.numel, d.chunks = offsets.data_ptr(), numel.data_ptr(), chunks.data_ptr()
                    d.caution_count = b.caution_scratch().data_ptr() if group["caution"] else None
                    d.n_chunks, d.n_tensors = n_chunks, len(b.params)
                    d.flags = flags
                    d.param_fmt = _lib.ECC_FMT[pecc] if pecc else _PLAIN_FMT[b.param_dtype]
                    d.neg_lr, d.one_minus_decay_lr = neg_lr, omdl
                    d.rng_mode, d.step, d.seed = self._rng_mode(), int(step) & 0xFFFFFFFF, self.rng_seed
                    _lib.check(L.hb_update_param(d, stream), "hb_update_param")
        self._last_launch = (None, keep)


class MuonAdamW(Muon, FirstOrder):
    """MuonAdamW with HeavyBall's signature (heavyball/__init__.py:475-540): parameters with two or more dimensions take
    the Muon chain (Nesterov-EMA momentum -> Newton-Schulz), the others ``scale_by_adam`` -> ``update_param_``.

    The un-fused ``scale_by_adam`` writes its result into the update buffer, which has the gradient's dtype; for fp32
    gradients that is the same arithmetic as the fused Adam step, so the vectors run on ``hb_fused_step`` under the
    state names of the un-fused transform.  bf16 gradients on the vector route take the step kernel's update-only mode,
    which rounds the update to bf16 as that buffer does, and ``hb_update_param`` after it (fp16 gradients likewise, with
    casts for roundings).
    State names and initialisation sets follow the reference's index walk with the route in place
    (``nesterov_ema_momentum_4`` with {2, 3, 4}, ``exp_avg_exp_avg_4`` under ``nesterov=False``; ``scale_by_adam_exp_avg_0`` /
    ``_exp_avg_sq_0`` with {0}; ``mars_mars_old_grad_6`` and a 6 in both sets under ``mars``).  ``ecc`` / ``storage_dtype`` apply
    to the state of both routes.  ``gradient_clipping`` / ``update_clipping`` act on the tensors of both routes at once, as the
    reference's chain places them around the route: a norm over the whole group is one norm over matrices and vectors.
    """

    KEY = "nesterov_ema_momentum_4"
    INIT = frozenset({2, 3, 4})
    _algo = _lib.ALGO_ADAM
    _fn_name = "scale_by_adam"
    _unfused_for_narrow_grads = True

    def __init__(self, params, lr=0.0025, betas=(0.9, 0.99), eps=1e-8, weight_decay=0, cautious_weight_decay: bool = False,
                 warmup_steps=0, multi_tensor: bool = True, storage_dtype: str = "float32", mars: bool = False,
                 caution: bool = False, mars_gamma: float = 0.0025, gradient_clipping=use_default, update_clipping=use_default,
                 palm: bool = use_default, beta2_scale: float = 0.8, nesterov: bool = True, compile_step: bool = use_default,
                 promote: bool = use_default, ecc: Optional[str] = None, param_ecc: Optional[str] = None, orig_shapes=None,
                 **kwargs):  # fmt: skip
        super().__init__(params, lr=lr, betas=betas, eps=eps, weight_decay=weight_decay, cautious_weight_decay=cautious_weight_decay,
                         warmup_steps=warmup_steps, multi_tensor=multi_tensor, storage_dtype=storage_dtype, mars=mars, caution=caution,
                         mars_gamma=mars_gamma, gradient_clipping=gradient_clipping, update_clipping=update_clipping, palm=palm,
                         beta2_scale=beta2_scale, nesterov=nesterov, compile_step=compile_step, promote=promote, ecc=ecc,
                         param_ecc=param_ecc, orig_shapes=orig_shapes, **kwargs)  # fmt: skip
        if not nesterov:  # heavyball/__init__.py:527-529: exp_avg heads the matrix route instead
            self.KEY = "exp_avg_exp_avg_4"
        for group in self.param_groups:  # the reference's MuonAdamW has no such argument (heavyball/__init__.py:499-523)
            group.pop("heavyball_momentum", None)
        self.defaults.pop("heavyball_momentum", None)

    def _route(self, p) -> int:
        return 1 if p.ndim >= 2 else 0

    def _run_group(self, gi, group, active):
        # the two routes side by side: a clip (heavyball/chainable.py:2696-2701 puts both clips around the route) acts on the
        # tensors of both at once, so a norm over the whole group spans matrices and vectors
        matrices = [(p, g) for p, g in active if p.ndim >= 2]
        vectors = [(p, g) for p, g in active if p.ndim < 2]
        gens = []
        if matrices:
            gens.append(Muon._run_group_gen(self, gi, group, matrices))
        if vectors:
            gens.append(FirstOrder._run_group_gen(self, gi, group, vectors))
        self._run_gens(gens)


class SplitOpt:
    """heavyball.SplitOpt (heavyball/__init__.py:1721-1762): delegates parameter groups to different optimizers.

        opt = SplitOpt([{"params": matrices, "optimizer": Muon, "lr": 0.02}, {"params": vectors, "optimizer": AdamW, "lr": 1e-3}])
    """

    def __init__(self, specs):
        self.optimizers = []
        for spec in specs:
            spec = dict(spec)
            params = list(spec.pop("params"))
            if params:
                self.optimizers.append(spec.pop("optimizer")(params, **spec))
        if not self.optimizers:
            raise ValueError("No optimizers created")

    @property
    def param_groups(self):
        return [g for opt in self.optimizers for g in opt.param_groups]

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        for opt in self.optimizers:
            opt.step()
        return loss

    def zero_grad(self, set_to_none: bool = True):
        for opt in self.optimizers:
            opt.zero_grad(set_to_none=set_to_none)

    def state_dict(self):
        return {"optimizers": [opt.state_dict() for opt in self.optimizers]}

    def load_state_dict(self, state_dict):
        if len(state_dict["optimizers"]) != len(self.optimizers):
            raise ValueError("state_dict holds a different number of optimizers")
        for opt, s in zip(self.optimizers, state_dict["optimizers"]):
            opt.load_state_dict(s)

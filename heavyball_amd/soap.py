"""SOAP (heavyball/__init__.py:839-909) on the HIP kernels.

Per parameter (viewed with the reference's dimension merging, heavyball/utils.py:240-272; two dimensions in the usual case)
the step is ``Ql^T G Qr`` -> Adam in the rotated basis -> ``Ql P Qr^T`` -> parameter update, plus the factor EMAs
``G G^T`` / ``G^T G``; a view that keeps more than two dimensions gets one rotation and one factor per dimension;
every product runs on ``hb_gemm_f32``, the Adam part on ``hb_adam_precond``, the parameter update on ``hb_update_param``.
The eigenbasis is initialised on the first step (which performs no parameter update) with ``torch.linalg.eigh``, one solve
per matrix on its smaller side with the other side's basis derived from it (``SOAP._first_bases``), and
refreshed with one power-iteration step + a QR factorisation when the schedule fires (heavyball/utils.py:829-900,
:986-1038, :3494-3500).  The QR runs on ``hb_orthonormalize_f32`` (block Gram-Schmidt on the GEMM kernel; its Q equals
Householder's up to column signs, which the step is invariant to) and falls back to ``torch.linalg.qr`` when a factor is
numerically rank-deficient; ``eigh`` stays in torch.

With ``split`` a parameter larger than max_precond_dim in some dimension is preconditioned block by block, every block with a
state of its own under ``state[p][k]`` (heavyball/utils.py:274-286, :1612-1623); what the chain keeps or counts outside the
preconditioner (MARS' old gradient, the correction of an ECC parameter, caution's count, the per-tensor norms of the clips) is
per block then as well.

State layout of the reference: ``scale_by_soap_exp_avg_2`` / ``scale_by_soap_exp_avg_sq_2`` with a leading bucket
dimension of 1, ``scale_by_soap_Q_3`` / ``scale_by_soap_GG_3`` as lists with one ``[1, d, d]`` tensor (or None) per dimension.
"""

import ctypes
from typing import Dict, List, Optional

import torch

from . import _lib
from .optim import HBOptimizer, _ECC_DTYPES, _PLAIN_FMT, beta_debias, build_defaults, current_stream_ptr, debiased_weights, f32, mars_weights, use_default

_GGT_CHUNK = 4096  # rows per independent piece of a long tensor's factor update (SOAP._update_ggt)
K_OLD = "mars_mars_old_grad_5"  # MARS' guard, three places behind the transform's in the reference's index walk
K_M, K_V, K_Q, K_GG = "scale_by_soap_exp_avg_2", "scale_by_soap_exp_avg_sq_2", "scale_by_soap_Q_3", "scale_by_soap_GG_3"


def merged_shape(shape, max_precond_dim: int):
    """heavyball/utils.py:240-272 (split=False): merge trailing dimensions while their product stays <= max_precond_dim."""
    new_shape, cum = [], 1
    for s in list(shape[1:])[::-1]:
        t = cum * s
        if t > max_precond_dim:
            if cum > 1:
                new_shape.append(cum)
                cum = s
            else:
                new_shape.append(s)
                cum = 1
        else:
            cum = t
    if cum > 1:
        new_shape.append(cum)
    return [shape[0], *new_shape[::-1]] if len(shape) else []


def split_blocks(shape, max_precond_dim: int):
    """heavyball/utils.py:274-286 (``dim_merger`` with split=True) as index arithmetic: None when no dimension of the merged view
    exceeds max_precond_dim, else one ``(slices into the merged view, shape of the block)`` per block.  Every oversized dimension is
    cut into runs of max_precond_dim (the last one shorter); the blocks are ordered with the cuts of the last such dimension
    outermost; dimensions of size one in the merged view are dropped from a block, whose remaining shape is merged again."""
    import itertools

    merged = merged_shape(shape, max_precond_dim) if len(shape) else []
    cuts = [[(a, min(a + max_precond_dim, sh)) for a in range(0, sh, max_precond_dim)] if sh > max_precond_dim else [(0, sh)] for sh in merged]
    if all(len(c) == 1 for c in cuts):
        return None
    out = []
    for combo in itertools.product(*reversed(cuts)):
        spans = combo[::-1]  # back in dimension order
        kept = [b - a for (a, b), sh in zip(spans, merged) if sh != 1]
        out.append((tuple(slice(a, b) for a, b in spans), merged_shape(kept, max_precond_dim) if kept else []))
    return out


class _Gemm:
    """Thin caller of hb_gemm_f32 on contiguous 2-D fp32 tensors.

    Between ``defer()`` and ``stop()`` the products are collected instead of launched, and ``flush()`` issues them through
    hb_gemm_f32_grouped: the products of different tensors (``owner``) are independent and share launches, the n-th product
    asked for on behalf of one owner since the last flush runs after that owner's (n-1)-th.  Nothing but another collected
    product may read a collected product's result before the flush."""

    def __init__(self, device):
        self.L = _lib.lib()
        self.device = device
        self.queue = None  # level -> [(A, B, C, M, N, K, ta, tb, flags, alpha, beta)] while deferring
        self.owner = None
        self._level: Dict[object, int] = {}
        self._then: List = []

    def defer(self):
        self.queue, self._level = {}, {}

    def then(self, fn):
        """Runs ``fn`` once the products asked for so far have been issued: at once, or after the next flush while deferring."""
        if self.queue is None:
            fn()
        else:
            self._then.append(fn)

    def stop(self):
        self.flush()
        self.queue = None

    def flush(self):
        if not self.queue and not self._then:
            return
        stream = current_stream_ptr(self.device)
        for level in sorted(self.queue):
            by_orientation: Dict[tuple, List] = {}
            for call in self.queue[level]:
                by_orientation.setdefault((call[6], call[7]), []).append(call)
            for (ta, tb), calls in by_orientation.items():
                n = len(calls)
                ptr = lambda k: (ctypes.c_void_p * n)(*[c[k].data_ptr() for c in calls])  # noqa: E731
                i64 = lambda vals: (ctypes.c_int64 * n)(*vals)  # noqa: E731
                _lib.check(self.L.hb_gemm_f32_grouped(n, ptr(0), ptr(1), ptr(2), i64([c[3] for c in calls]), i64([c[4] for c in calls]),
                                                      i64([c[5] for c in calls]), i64([c[0].shape[1] for c in calls]),
                                                      i64([c[1].shape[1] for c in calls]), i64([c[4] for c in calls]), int(ta), int(tb),
                                                      (ctypes.c_int32 * n)(*[c[8] for c in calls]), (ctypes.c_float * n)(*[c[9] for c in calls]),
                                                      (ctypes.c_float * n)(*[c[10] for c in calls]), stream), "hb_gemm_f32_grouped")  # fmt: skip
        self.queue, self._level = {}, {}
        hooks, self._then = self._then, []
        for fn in hooks:
            fn()

    def barrier(self):
        """What the current owner asks for next waits for everything it has asked for so far (``independent`` products included)."""
        if self.queue is not None:
            self._level[self.owner] = self._level.get(self.owner, 0) + 1

    def __call__(self, A, B, C, ta=False, tb=False, accumulate=False, alpha=1.0, beta=0.0, symmetric=False, independent=False):
        """``independent``: the product neither reads nor overwrites what the owner's last product wrote, and may share its launch."""
        M = A.shape[1] if ta else A.shape[0]
        K = A.shape[0] if ta else A.shape[1]
        N = B.shape[0] if tb else B.shape[1]
        assert (B.shape[1] if tb else B.shape[0]) == K and tuple(C.shape) == (M, N)
        assert A.is_contiguous() and B.is_contiguous() and C.is_contiguous() and A.dtype == B.dtype == C.dtype == torch.float32
        flags = (_lib.GEMM_ACCUMULATE if accumulate else 0) | (_lib.GEMM_SYMMETRIC if symmetric else 0)
        if self.queue is not None:
            level = self._level.get(self.owner, 0)
            if not independent:
                self._level[self.owner] = level + 1
            self.queue.setdefault(level, []).append((A, B, C, M, N, K, ta, tb, flags, alpha, beta))
            return C
        _lib.check(self.L.hb_gemm_f32(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, A.shape[1], B.shape[1], N, int(ta), int(tb),
                                      flags, alpha, beta, current_stream_ptr(self.device)), "hb_gemm_f32")  # fmt: skip
        return C


class _Ortho:
    """One ``hb_orthonormalize_f32`` call in flight: the matrix, its work space and its status word."""

    def __init__(self, A: torch.Tensor, status: Optional[torch.Tensor] = None):
        assert A.dim() == 2 and A.is_contiguous() and A.dtype == torch.float32 and A.shape[1] <= A.shape[0]
        self.A = A
        m, n = A.shape
        nb = ctypes.c_int64()
        _lib.check(_lib.lib().hb_orthonormalize_workspace_bytes(m, n, ctypes.byref(nb)), "hb_orthonormalize_workspace_bytes")
        self.ws = torch.empty(nb.value, dtype=torch.uint8, device=A.device)
        self.status = torch.empty(1, dtype=torch.int32, device=A.device) if status is None else status

    def launch(self, stream: Optional[torch.cuda.Stream] = None):
        A = self.A
        sp = current_stream_ptr(A.device) if stream is None else stream.cuda_stream
        with torch.cuda.device(A.device):
            _lib.check(_lib.lib().hb_orthonormalize_f32(A.data_ptr(), A.shape[0], A.shape[1], A.shape[1], self.ws.data_ptr(), self.ws.numel(),
                                                        self.status.data_ptr(), sp), "hb_orthonormalize_f32")  # fmt: skip


def launch_orthonormalize(jobs: List[_Ortho], stream: Optional[torch.cuda.Stream] = None):
    """Starts the factorisations of ``jobs``: matrices of one shape go through ``hb_orthonormalize_f32_batched`` in groups of
    up to ``_lib.ORTHO_MAX_BATCH`` (every launch of the chain then covers the whole group), the rest one by one."""
    L = _lib.lib()
    groups: Dict[tuple, List[_Ortho]] = {}
    for j in jobs:
        groups.setdefault((tuple(j.A.shape), j.A.device, j.A.data_ptr() % 16), []).append(j)
    for (shape, dev, _), members in groups.items():
        sp = current_stream_ptr(dev) if stream is None else stream.cuda_stream
        with torch.cuda.device(dev):
            for k in range(0, len(members), _lib.ORTHO_MAX_BATCH):
                part = members[k : k + _lib.ORTHO_MAX_BATCH]
                if len(part) == 1:
                    part[0].launch(stream)
                    continue
                n = len(part)
                q = (ctypes.c_void_p * n)(*[j.A.data_ptr() for j in part])
                ws = (ctypes.c_void_p * n)(*[j.ws.data_ptr() for j in part])
                st = (ctypes.c_void_p * n)(*[j.status.data_ptr() for j in part])
                _lib.check(L.hb_orthonormalize_f32_batched(n, q, shape[0], shape[1], shape[1], ws, min(j.ws.numel() for j in part), st, sp),
                           "hb_orthonormalize_f32_batched")  # fmt: skip


def orthonormalize_(A: torch.Tensor) -> bool:
    """Replaces the columns of the contiguous fp32 matrix ``A`` [m, n] (n <= m) by the Q factor of its thin QR
    decomposition (positive diagonal of R) with ``hb_orthonormalize_f32``.  Returns False when a panel was numerically
    rank-deficient; ``A`` then holds garbage and the caller must redo the factorisation another way."""
    job = _Ortho(A)
    job.launch()
    return int(job.status.item()) == 0


class SOAP(HBOptimizer):
    """SOAP with HeavyBall's signature (heavyball/__init__.py:875-909)."""

    def __init__(self, params, lr: float = 3e-3, betas=(0.9, 0.95), shampoo_beta: float = 0.95, eps: float = 1e-8,
                 weight_decay: float = 0.01, cautious_weight_decay: bool = False, precondition_frequency: int = 2,
                 max_precond_dim: int = 2048, merge_dims: bool = True, precondition_1d: bool = False, warmup_steps: int = 0,
                 split: bool = False, multi_tensor: bool = True, mars: bool = False, caution: bool = False,
                 mars_gamma: float = 0.0025, palm: bool = use_default, precond_scheduler=(1 / 3, 9), beta2_scale: float = 0.8,
                 use_precond_schedule: bool = use_default, gradient_clipping=use_default, update_clipping=use_default,
                 storage_dtype: str = "float32", precond_grad_accum: bool = False, compile_step: bool = use_default,
                 promote: bool = use_default, ecc: Optional[str] = None, param_ecc: Optional[str] = None, orig_shapes=None, **kwargs):  # fmt: skip
        params, defaults = build_defaults(locals())
        if defaults.pop("use_precond_schedule") not in (use_default, False):
            # the reference cannot run it either: heavyball/utils.py:3497 hands the schedule a python int and :2411 calls .clamp on it
            raise NotImplementedError("SOAP: use_precond_schedule (the reference's own schedule fails on its first call)")
        del defaults["precond_scheduler"]
        self.precond_schedule = 1 / defaults.pop("precondition_frequency")  # heavyball/__init__.py:842-858
        # precond_grad_accum is read by PSGD's guard only (heavyball/chainable.py:304-345): SOAP's chain ignores it, and so does this
        self._block_copies = []  # per-block state entries that cannot be views of their slab role: refreshed after every step
        super().__init__(params, defaults, gradient_clipping, update_clipping, palm)

    def _adopt_group(self, gi, group):
        super()._adopt_group(gi, group)
        if group.get("param_ecc"):  # heavyball/chainable.py:2438-2444: one correction tensor per view of the parameter
            for b in self._buckets[gi]:
                for i, p in enumerate(b.params):
                    self._expose_blocks(group, b, i, p, ("param::ecc",))

    # -- split: state outside the preconditioner, per block ----------------------------------------------------------------
    # With split the reference runs its whole chain per block (heavyball/utils.py:1612-1623), so MARS' old gradient, the
    # correction of an ECC parameter, caution's count and the per-tensor norms of the clips are per block.  The kernels keep
    # working on whole parameters: the old gradient and the correction stay slab roles in the parameter's own layout (both are
    # elementwise), and ``state[p][k]`` shows block k of them; counts and norms per block are taken with torch on block views.
    def _blocks_of(self, group, p):
        """None, or ``[(slices into the merged view, block shape)]`` for a parameter that split cuts up."""
        if not (group.get("merge_dims", True) and group.get("split") and p.dim() > 0):
            return None
        return split_blocks(p.shape, group["max_precond_dim"])

    def _expose_blocks(self, group, b, i, p, keys, value=None):
        """``state[p][k][key]`` = block k of the slab role ``key`` for a parameter that split cuts up (True), nothing otherwise
        (False): a view where the block's own shape can be one, else a copy that ``_refresh_block_copies`` keeps current.
        ``value``: {key: {k: tensor}} to write into the role first (a loaded checkpoint)."""
        blocks = self._blocks_of(group, p)
        if blocks is None:
            return False
        merged = merged_shape(p.shape, group["max_precond_dim"])
        self._block_copies = [c for c in self._block_copies if not (c[2] is b and c[3] == i and c[1] in keys)]
        for k, (where, bshape) in enumerate(blocks):
            st = self.state[p].setdefault(k, {})
            for key in keys:
                if not b.slab.has(key):
                    continue
                part = b.slab.view(key, i).reshape(merged)[where]
                if value is not None and k in value.get(key, {}):
                    part.copy_(value[key][k].to(part.dtype).reshape(part.shape))
                try:
                    st[key] = part.view(bshape or [1])
                except RuntimeError:  # the block's shape merges dimensions that are strided in the parameter
                    st[key] = part.reshape(bshape or [1])
                    self._block_copies.append((st, key, b, i, tuple(merged), where, tuple(bshape or [1])))
        return True

    def _refresh_block_copies(self):
        for st, key, b, i, merged, where, bshape in self._block_copies:
            st[key] = b.slab.view(key, i).reshape(merged)[where].reshape(bshape)

    @staticmethod
    def _per_block(view, blocks, fn):
        """``fn(block)`` in place on every block of a tensor's merged view."""
        for where, _ in blocks:
            fn(view[where])

    @staticmethod
    def _clip_block_(kind):
        """heavyball/utils.py:3226-3262 on one view, in place: the per-tensor clips, which split takes per block."""
        def clip(x):
            norm = x.norm() if kind == "l2_clip_" else x.square().mean().sqrt()
            x.mul_(1.0 / norm.clamp(min=1.0))  # clip_at = 1: clip_at / max(norm, clip_at, eps)
        return clip

    def _run_group(self, gi, group, active):
        active = [(p, g) for p, g in active if p.numel() > 0]  # an empty tensor has nothing to precondition or update
        if not active:
            return
        L = _lib.lib()
        step = group["step"]
        lr = f32(group["lr"])
        beta1, beta2 = self._betas(group, step)
        adam_step = step - 1  # heavyball/chainable.py:1270
        max_dim = group["max_precond_dim"]
        decay = group["weight_decay"]
        omdl, neg_lr = float(1 - decay * lr), float(-lr)
        flags = (_lib.FLAG_CAUTION if group["caution"] else 0) | (_lib.FLAG_CAUTIOUS_WD if group.get("cautious_weight_decay", False) else 0)
        is_precond = bool(group["is_preconditioning"])
        pecc = group.get("param_ecc")
        if group.get("ecc"):
            mom_prim, mom_corr = _ECC_DTYPES[group["ecc"]]
            mom_fmt = _lib.ECC_FMT[group["ecc"]]
        else:
            mom_prim, mom_corr = getattr(torch, group.get("storage_dtype", "float32")), None
            mom_fmt = _PLAIN_FMT[mom_prim]

        per_bucket: Dict[int, List] = {}
        for p, g in active:
            b, i = self._find_bucket(gi, p)
            per_bucket.setdefault(id(b), [b, []])[1].append((i, p, g))
        raw: Dict[int, List] = {}
        gdts: Dict[int, List] = {}  # the dtype of each tensor's update buffer: its gradient's (fp32 under promote)
        keep_given = []
        for key, (b, items) in per_bucket.items():
            if b.device.type != "cuda":
                raise _lib.HbError("the optimizer step runs on the GPU only: parameters must live on a CUDA/HIP device")
            self._check_home(b, items)
            # 16-bit gradients (without promote): the preconditioner itself promotes what it is handed (heavyball/chainable.py:1261,
            # :1248), so the gradient's values go through it as fp32; what stays 16-bit is the update buffer ahead of it (MARS and a
            # gradient clip round into it) and the factors and bases, which are created in the gradient's dtype (gdts, see precondition)
            given = []
            for _, _, g in items:
                if g.is_sparse:
                    raise NotImplementedError("sparse gradients")
                if g.dtype not in _PLAIN_FMT or (self.promote and g.dtype != torch.float32):
                    g = g.float()
                if g.device != b.device or not g.is_contiguous() or g.data_ptr() % 16:
                    g = g.to(b.device).clone(memory_format=torch.contiguous_format)
                given.append(g)
            gdts[key] = [g.dtype for g in given]
            raw[key] = [g if g.dtype == torch.float32 else g.float() for g in given]
            if group.get("mars"):
                # heavyball/chainable.py:642-647 heads the chain and writes the corrected gradient over the gradient itself: a
                # pass of its own leaves it in the fp32 role "_clip", which then stands for the gradient everywhere below
                # mars_old_grad is stored like the moments (zero_guard with the group's storage, heavyball/chainable.py:277-301)
                b.slab.role(K_OLD, mom_prim)
                if mom_corr is not None:
                    b.slab.role(K_OLD + "::ecc", mom_corr)
                for (i, p, _), g32 in zip(items, raw[key]):
                    st = self._state0(p)
                    if K_OLD not in st:
                        if self._expose_blocks(group, b, i, p, (K_OLD, K_OLD + "::ecc")):  # split: one old gradient per block
                            for bst in self.state[p].values():
                                if isinstance(bst, dict) and K_OLD in bst:
                                    bst.setdefault("is_initialized", set()).add(5)
                            continue
                        st[K_OLD] = b.slab.view(K_OLD, i)
                        if mom_corr is not None:
                            st[K_OLD + "::ecc"] = b.slab.view(K_OLD + "::ecc", i)
                        st.setdefault("is_initialized", set()).add(5)
                for gdt in sorted(set(gdts[key]), key=str):  # the corrected gradient is rounded into the gradient's dtype
                    lst = sorted(((i, g) for (i, _, _), g in zip(items, given) if g.dtype == gdt), key=lambda t: t[0])
                    self._mars_prologue(L, group, b, lst, gdt, step, *mars_weights(group), mom_fmt, K_OLD)
                keep_given.append(given)
                raw[key] = [b.slab.view("_clip", i) for i, _, _ in items]
                if self.gradient_clipping is not None:
                    # the clip below rewrites the role in place; what stands for the gradient (the first factors of a tensor's
                    # first step, heavyball/chainable.py:1235-1238, and caution's sign test) is the corrected gradient before it
                    raw[key] = [(v.clone() if K_M not in self._state0(p) or group["caution"] else v) for v, (_, p, _) in zip(raw[key], items)]
        if self.gradient_clipping is not None:
            # heavyball/chainable.py:2696-2699: the clip acts on the update; the gradient itself still initialises the
            # factors (:1235-1238) and is what caution compares against
            # a norm per tensor is a norm per block under split (heavyball/utils.py:1612-1623): those tensors are clipped here,
            # block by block, and left out of the kernels' clip
            own = self.gradient_clipping in ("l2_clip_", "rmsnorm_clip_")
            work, own_narrow = [], []
            for key, (b, items) in per_bucket.items():
                b.slab.role("_clip", torch.float32)
                lists: Dict[torch.dtype, List] = {}
                for (i, p, _), g32, gdt in zip(items, raw[key], gdts[key]):
                    blocks = self._blocks_of(group, p) if own else None
                    if blocks is None:
                        lists.setdefault(gdt, []).append((i, g32))
                        continue
                    view = b.slab.view("_clip", i)
                    if not group.get("mars"):  # otherwise the MARS pass has left the gradient there
                        view.copy_(g32)
                    self._per_block(view.reshape(merged_shape(p.shape, max_dim)), blocks, self._clip_block_(self.gradient_clipping))
                    if gdt != torch.float32:
                        own_narrow.append((b, i, gdt))
                for gdt, lst in lists.items():
                    work.append((b, sorted(lst, key=lambda t: t[0]), gdt))
            clipped_role = {}
            if work:
                for (b, _, gdt), res in zip(work, self._clip_gradients(L, group, work, step, gathered=bool(group.get("mars")))):
                    clipped_role[(id(b), gdt)] = res[0]
            for b, i, gdt in own_narrow:  # the clipped values go back into the 16-bit update buffer (heavyball/utils.py:3231)
                view = b.slab.view("_clip", i)
                if gdt == torch.bfloat16:
                    narrow = torch.empty_like(view, dtype=torch.bfloat16)
                    with torch.cuda.device(b.device):
                        _lib.check(L.hb_sr_bf16(view.data_ptr(), narrow.data_ptr(), view.numel(), self._rng_mode(), self.rng_seed,
                                                int(step) & 0xFFFFFFFF, _lib.STREAM_CLIP, int(b.slab.offsets_np[i]), current_stream_ptr(b.device)),
                                   "hb_sr_bf16")  # fmt: skip
                    view.copy_(narrow)
                else:
                    view.copy_(view.to(gdt))
        pending = []  # parameter updates, launched once the (optionally clipped) update of the whole group is there
        for key, (b, items) in per_bucket.items():
            b.slab.role("_update", torch.float32)
            gemm = _Gemm(b.device)
            stream = current_stream_ptr(b.device)
            updated, keep, refresh, first = [], [], [], []
            with torch.cuda.device(b.device):
                def precondition(st, G0, G, out, base, fdt):
                    """One tensor or block: G0 the gradient, G the update that goes through the preconditioner, both in the merged
                    view (fp32 values); the preconditioned update lands in ``out``.  False on the first step, which only initialises.
                    ``fdt``: the gradient's dtype, which the factors and bases created here take (heavyball/utils.py:1381, :996)."""
                    if K_M not in st:  # first step: initialise, no update (heavyball/chainable.py:372-377, utils.py:1362-1388)
                        for km in (K_M, K_V):  # zero_guard with the group's storage (heavyball/chainable.py:277-301)
                            st[km] = torch.zeros((1, *G.shape), dtype=mom_prim, device=b.device)
                            if mom_corr is not None:
                                st[km + "::ecc"] = torch.zeros((1, *G.shape), dtype=mom_corr, device=b.device)
                        GG: List[Optional[torch.Tensor]] = []
                        if G.numel() > 1 and (G.dim() >= 2 or group.get("precondition_1d")):  # heavyball/utils.py:1370
                            for sh in G.shape:
                                GG.append(None if (sh > max_dim or sh == 1) else torch.zeros((1, sh, sh), dtype=torch.float32, device=b.device))
                        else:
                            GG.append(None)
                        self._update_ggt(gemm, G0, GG, 1.0, 0.0)  # beta = 0: a = 1
                        if fdt != torch.float32:
                            # 16-bit factors: the first one is the rounded product itself (the reference's contraction of a 16-bit
                            # gradient returns that dtype, utils.py:1387); the basis below comes from the stored values and is cast (:1003)
                            GG = [None if m is None else m.to(fdt) for m in GG]
                        st[K_GG] = GG
                        first.append((st, G0, GG, fdt, base))  # the bases of every tensor's first step are found together, below
                        st.setdefault("is_initialized", set()).update({0, 2, 3})
                        return False
                    GG, Q = self._factors32(st)
                    gp = self._project(gemm, G, Q, back=False)
                    a1, oma1 = debiased_weights(beta1, adam_step)
                    a2, oma2 = debiased_weights(beta2, adam_step)
                    if gp is G:
                        gp = G.clone()
                    # moments kept as bf16 or as an ECC pair are widened to fp32 for the step and written back through the
                    # codec; the update comes from the fp32 values before that rounding, as in the reference (utils.py:1842-1849)
                    m32, v32 = self._widen(L, st, K_M, mom_fmt, stream), self._widen(L, st, K_V, mom_fmt, stream)
                    _lib.check(L.hb_adam_precond(m32.data_ptr(), v32.data_ptr(), gp.data_ptr(), gp.data_ptr(), gp.numel(), a1, oma1,
                                                 a2, oma2, float(f32(group["eps"])), stream), "hb_adam_precond")  # fmt: skip
                    if mom_fmt != _lib.FMT_F32:
                        self._narrow(L, st, K_M, m32, mom_fmt, _lib.STREAM_EXP_AVG, step, base, stream)
                        self._narrow(L, st, K_V, v32, mom_fmt, _lib.STREAM_EXP_AVG_SQ, step, base, stream)
                    back = self._project(gemm, gp, Q, back=True, out=out)
                    if back is not out:  # no basis at all, or the last product went through a moved dimension
                        out.copy_(back)
                    sb = beta_debias(group["shampoo_beta"], step)  # heavyball/chainable.py:1244: python float and int64 0-d tensor
                    a = 1 - sb
                    a = a.to(torch.float32) if isinstance(a, torch.Tensor) else f32(a)
                    self._update_ggt(gemm, G, GG, float(a), float(1 - a))
                    self._store_factors(L, st, K_GG, GG, _lib.STREAM_SOAP_GG, step, base, stream)
                    if is_precond:
                        if mom_fmt == _lib.FMT_F32:
                            refresh.append((GG, Q, st[K_M], st, base))
                        else:  # the rotation reads exp_avg as stored (heavyball/utils.py:883) and writes it back through the codec
                            refresh.append((GG, Q, self._widen(L, st, K_M, mom_fmt, stream), st, base))
                    return True

                # Tensors beyond their first step whose view has at most two dimensions go through the preconditioner stage by
                # stage, all of them together, so that each stage's products share launches (hb_gemm_f32_grouped): on a model of
                # many mid-sized matrices one product at a time leaves most of the chip idle.  The arithmetic per tensor is that of
                # ``precondition``.  A batch ends when its temporaries reach a quarter of a GiB-element.
                staged: List[dict] = []
                staged_elems = [0]

                def run_staged():
                    if not staged:
                        return
                    gemm.defer()
                    for w in staged:  # into the eigenbasis
                        gemm.owner = id(w)
                        w["GG"], w["Q"] = self._factors32(w["st"])
                        w["gp"] = self._project(gemm, w["G"], w["Q"], back=False)
                    gemm.flush()
                    a1, oma1 = debiased_weights(beta1, adam_step)
                    a2, oma2 = debiased_weights(beta2, adam_step)
                    adam = []  # Adam there, for all of them in one launch
                    for w in staged:
                        st, gp = w["st"], w["gp"]
                        src = gp
                        if gp is w["G"]:  # no basis at all (a vector): Adam reads the update and writes the result where it belongs
                            gp = w["gp"] = w["out"]
                        w["m32"], w["v32"] = self._widen(L, st, K_M, mom_fmt, stream), self._widen(L, st, K_V, mom_fmt, stream)
                        adam.append((w["m32"].data_ptr(), w["v32"].data_ptr(), src.data_ptr(), gp.data_ptr(), gp.numel()))
                    n = len(adam)
                    cols = [(ctypes.c_void_p * n)(*[t[k] for t in adam]) for k in range(4)]
                    _lib.check(L.hb_adam_precond_grouped(n, *cols, (ctypes.c_int64 * n)(*[t[4] for t in adam]), a1, oma1, a2, oma2,
                                                         float(f32(group["eps"])), stream), "hb_adam_precond_grouped")  # fmt: skip
                    if mom_fmt != _lib.FMT_F32:
                        for w in staged:
                            self._narrow(L, w["st"], K_M, w["m32"], mom_fmt, _lib.STREAM_EXP_AVG, step, w["base"], stream)
                            self._narrow(L, w["st"], K_V, w["v32"], mom_fmt, _lib.STREAM_EXP_AVG_SQ, step, w["base"], stream)
                    for w in staged:  # and back
                        gemm.owner = id(w)
                        w["back"] = self._project(gemm, w["gp"], w["Q"], back=True, out=w["out"])
                    gemm.flush()
                    sb = beta_debias(group["shampoo_beta"], step)  # heavyball/chainable.py:1244: python float and int64 0-d tensor
                    a = 1 - sb
                    a = a.to(torch.float32) if isinstance(a, torch.Tensor) else f32(a)
                    for w in staged:  # the factors take the update's outer products
                        if w["back"] is not w["out"]:
                            w["out"].copy_(w["back"])
                        gemm.owner = id(w)
                        self._update_ggt(gemm, w["G"], w["GG"], float(a), float(1 - a))
                    gemm.stop()
                    for w in staged:
                        st = w["st"]
                        self._store_factors(L, st, K_GG, w["GG"], _lib.STREAM_SOAP_GG, step, w["base"], stream)
                        if is_precond:
                            exp_avg = st[K_M] if mom_fmt == _lib.FMT_F32 else self._widen(L, st, K_M, mom_fmt, stream)
                            refresh.append((w["GG"], w["Q"], exp_avg, st, w["base"]))
                        if w["after"] is not None:
                            w["after"]()
                    staged.clear()
                    staged_elems[0] = 0

                def take(st, G0, G, out, base, fdt, after):
                    """One tensor or block on its way through the preconditioner, staged with the others where that is possible;
                    ``after`` runs once its update is in ``out``.  False on the first step, which only initialises."""
                    if K_M not in st or G.dim() > 2 or not self.group_products:
                        done = precondition(st, G0, G, out, base, fdt)
                        if done and after is not None:
                            after()
                        return done
                    staged.append(dict(st=st, G=G, out=out, base=base, after=after))
                    staged_elems[0] += G.numel()
                    if staged_elems[0] >= 1 << 28:
                        run_staged()
                    return True

                for (i, p, g), g32, gdt in zip(items, raw[key], gdts[key]):
                    keep.append(g32)
                    # heavyball/utils.py:3726-3742: without merge_dims the parameter is taken as it is
                    merging = group.get("merge_dims", True)
                    shape = (merged_shape(p.shape, max_dim) if merging else list(p.shape)) if p.dim() > 0 else []
                    G0 = g32.reshape(shape) if shape else g32.reshape(1)  # the gradient
                    G = G0  # the update
                    if self.gradient_clipping is not None:
                        role = clipped_role.get((id(b), gdt))  # a 16-bit role where the kernels' clip rounded into one
                        if role is not None and role.dtype != torch.float32 and not (own and self._blocks_of(group, p) is not None):
                            G = b.slab.view("_clip16" if role.dtype == torch.bfloat16 else "_clip16h", i).float().reshape(G0.shape)
                        else:
                            G = b.slab.view("_clip", i).reshape(G0.shape)
                    out = b.slab.view("_update", i).view(G.shape)
                    blocks = split_blocks(p.shape, max_dim) if merging and group.get("split") and p.dim() > 0 else None
                    if blocks is None:
                        if take(self._state0(p), G0, G, out, int(b.slab.offsets_np[i]), gdt, None):
                            updated.append(i)
                        continue
                    # split: every block is preconditioned on its own, with its own state (heavyball/utils.py:274-286, :1612-1623);
                    # a block is a strided part of the parameter, so it is gathered, and its update scattered into the slab
                    done, start = False, int(b.slab.offsets_np[i])  # the blocks' moments take consecutive runs of the parameter's noise
                    for k, (where, bshape) in enumerate(blocks):
                        bshape = bshape or [1]
                        g0b = G0[where].contiguous().reshape(bshape)
                        gb = g0b if G is G0 else G[where].contiguous().reshape(bshape)
                        ob = torch.empty_like(gb)
                        scatter = lambda ob=ob, where=where, out=out: out[where].copy_(ob.reshape(out[where].shape))  # noqa: E731
                        if take(self.state[p].setdefault(k, {}), g0b, gb, ob, start, gdt, scatter):
                            done = True
                        start += gb.numel()
                    if done:
                        updated.append(i)
                run_staged()
                if first:
                    for (st, *_), Q in zip(first, self._first_bases_of([e[1:] for e in first])):
                        st[K_Q] = Q
                if refresh:
                    self._refresh(gemm, refresh)
                    for GG32, Q32, exp_avg, st, base in refresh:
                        if mom_fmt != _lib.FMT_F32:
                            self._narrow(L, st, K_M, exp_avg, mom_fmt, _lib.STREAM_SOAP_ROTATE, step, base, stream)
                        self._store_factors(L, st, K_Q, Q32, _lib.STREAM_SOAP_Q, step, base, stream)  # heavyball/utils.py:898-900
            if updated:
                pending.append((b, sorted(updated), items, keep))
        # tensors that split cuts up: their per-tensor update clip and caution's count are per block (torch on block views)
        cut = {}
        per_block_clip = self.update_clipping in ("l2_clip_", "rmsnorm_clip_")
        if group.get("split") and (per_block_clip or group["caution"]):
            for b, updated, items, keep in pending:
                for (i, p, _), g32 in zip(items, keep):
                    blocks = self._blocks_of(group, p) if i in updated else None
                    if blocks is not None:
                        cut[(id(b), i)] = (p, g32, blocks)
        if self.update_clipping is not None and pending:  # heavyball/chainable.py:2700-2701
            rest = [(b, [i for i in updated if not (per_block_clip and (id(b), i) in cut)]) for b, updated, _, _ in pending]
            rest = [(b, idx) for b, idx in rest if idx]
            clip_keep = self._clip_updates(L, rest) if rest else None
            if per_block_clip:
                for b, updated, _, _ in pending:
                    for i in updated:
                        if (id(b), i) in cut:
                            p, _, blocks = cut[(id(b), i)]
                            self._per_block(b.slab.view("_update", i).reshape(merged_shape(p.shape, max_dim)), blocks, self._clip_block_(self.update_clipping))
        else:
            clip_keep = None
        launches = []
        for b, updated, items, keep in pending:
            if group["caution"] and any((id(b), i) in cut for i in updated):
                # heavyball/utils.py:3652-3658 per block, ahead of the parameter update, which then runs without the flag
                for i in updated:
                    if (id(b), i) not in cut:
                        continue
                    p, g32, blocks = cut[(id(b), i)]
                    merged = merged_shape(p.shape, max_dim)
                    uview, gview = b.slab.view("_update", i).reshape(merged), g32.reshape(merged)
                    for where, _ in blocks:
                        u, g = uview[where], gview[where]
                        mask = torch.signbit(g) ^ torch.signbit(u)
                        u.masked_fill_(mask, 0)
                        u.mul_(mask.numel() / (mask.numel() - mask.sum()).clamp(min=1))
                plain = [i for i in updated if (id(b), i) not in cut]
                if plain:
                    launches.append((b, plain, items, keep, flags))
                launches.append((b, [i for i in updated if (id(b), i) in cut], items, keep, flags & ~_lib.FLAG_CAUTION))
            else:
                launches.append((b, updated, items, keep, flags))
        for b, updated, items, keep, flags in launches:
            with torch.cuda.device(b.device):
                offsets, numel = b.slab.meta()
                chunks, n_chunks = b.slab.chunks(tuple(updated))
                d = _lib.HbStepDesc()
                d.param, d.param_corr = b.slab.ptr("param"), b.slab.ptr("param::ecc")
                ptrs = [0] * len(b.params)
                for (i, _, _), g32 in zip(items, keep):
                    ptrs[i] = g32.data_ptr()
                table = b.grad_ptr_table("soap", ptrs)
                d.grad, d.grad_ptrs = None, table.data_ptr()
                d.exp_avg = b.slab.ptr("_update")
                d.offsets, d.numel, d.chunks = offsets.data_ptr(), numel.data_ptr(), chunks.data_ptr()
                d.caution_count = b.caution_scratch().data_ptr() if flags & _lib.FLAG_CAUTION else None
                d.n_chunks, d.n_tensors = n_chunks, len(b.params)
                d.flags, d.param_fmt, d.grad_fmt = flags, (_lib.ECC_FMT[pecc] if pecc else _PLAIN_FMT[b.param_dtype]), _lib.FMT_F32
                d.neg_lr, d.one_minus_decay_lr = neg_lr, omdl
                d.rng_mode, d.step, d.seed = self._rng_mode(), int(step) & 0xFFFFFFFF, self.rng_seed
                _lib.check(L.hb_update_param(d, current_stream_ptr(b.device)), "hb_update_param")
        self._refresh_block_copies()
        self._last_launch = (None, [k for *_, k in pending], clip_keep)

    def _rehome_state(self):
        """torch's ``load_state_dict`` casts floating-point state to the parameter's dtype: the moments go back to their storage
        dtype (their values are representable there, heavyball/chainable.py:2452-2484 does the same).  A tensor that needs no
        cast is handed over as it is, so a state_dict taken from a live optimizer in the same process would share its moments,
        factors and bases with this one: every state tensor of the preconditioner is copied."""
        super()._rehome_state()
        for gi, group in enumerate(self.param_groups):
            for p in group["params"]:
                if p not in self.state:
                    continue
                if self._blocks_of(group, p) is not None:
                    # state outside the preconditioner of a parameter that split cuts up: the loaded blocks go back into their
                    # slab roles (the parameter's own layout), and state[p][k] shows block k of the role again
                    keys = [k_ for k_ in (K_OLD, K_OLD + "::ecc", "param::ecc")
                            if any(isinstance(st, dict) and k_ in st for st in self.state[p].values())]  # fmt: skip
                    if keys:
                        b, i = self._find_bucket(gi, p)
                        for k_ in keys:
                            b.slab.role(k_, self._role_dtype(group, k_))
                        value = {k_: {bk: st[k_] for bk, st in self.state[p].items() if isinstance(st, dict) and k_ in st} for k_ in keys}
                        self._expose_blocks(group, b, i, p, keys, value=value)
                for st in self.state[p].values():  # block 0, and the further blocks of a split parameter
                    if not isinstance(st, dict):
                        continue
                    for key in (K_M, K_V, K_M + "::ecc", K_V + "::ecc"):
                        if isinstance(st.get(key), torch.Tensor):
                            st[key] = st[key].to(self._role_dtype(group, key), copy=True).contiguous()
                    for key in (K_Q, K_GG):  # in the dtype they come back in: torch's load has cast them to the parameter's
                        if isinstance(st.get(key), (list, tuple)):
                            st[key] = [None if t is None else t.to(t.dtype if t.dtype in _PLAIN_FMT else torch.float32, copy=True).contiguous()
                                       for t in st[key]]  # fmt: skip

    # -- pieces ----------------------------------------------------------------------------------------------------
    @staticmethod
    def _factors32(st):
        """The factors and bases of a state as the fp32 tensors the products run on: the stored ones, or - kept in a 16-bit
        dtype - fp32 copies of them for the length of the step."""
        widen = lambda ts: [t if t is None or t.dtype == torch.float32 else t.float() for t in ts]  # noqa: E731
        return widen(st[K_GG]), widen(st[K_Q])

    def _store_factors(self, L, st, key, values32, stream_id, step, base, stream):
        """``copy_stochastic_`` of freshly computed fp32 factors or bases into their 16-bit storage (heavyball/utils.py:1048,
        :898-900), side li with noise stream ``stream_id + 2 * li`` at the places ``base + e``; the fp32 copies then take the
        stored values again.  Nothing to do for fp32 storage, where ``values32`` are the stored tensors."""
        for li, (t, v) in enumerate(zip(st[key], values32)):
            if t is None or t is v:
                continue
            if t.dtype == torch.bfloat16:
                _lib.check(L.hb_sr_bf16(v.data_ptr(), t.data_ptr(), t.numel(), self._rng_mode(), self.rng_seed, int(step) & 0xFFFFFFFF,
                                        stream_id + 2 * li, base, stream), "hb_sr_bf16")  # fmt: skip
            else:
                t.copy_(v)
            v.copy_(t)

    def _widen(self, L, st, key, fmt, stream):
        """The moment ``st[key]`` as fp32: itself when stored so, else a decoded copy."""
        t = st[key]
        if fmt == _lib.FMT_F32:
            return t
        if fmt == _lib.FMT_BF16:
            return t.float()
        out = torch.empty(t.shape, dtype=torch.float32, device=t.device)
        _lib.check(L.hb_ecc_decode(t.data_ptr(), st[key + "::ecc"].data_ptr(), out.data_ptr(), t.numel(), fmt, stream), "hb_ecc_decode")
        return out

    def _narrow(self, L, st, key, value, fmt, stream_id, step, base, stream):
        """``copy_stochastic_`` of an fp32 moment into its bf16 or ECC storage (heavyball/utils.py:2363-2370, :1296-1311); the noise
        of element e is that of flat index ``base + e``, ``base`` being the parameter's offset in its slab."""
        t = st[key]
        if fmt == _lib.FMT_BF16:
            _lib.check(L.hb_sr_bf16(value.data_ptr(), t.data_ptr(), t.numel(), self._rng_mode(), self.rng_seed, int(step) & 0xFFFFFFFF,
                                    stream_id, base, stream), "hb_sr_bf16")  # fmt: skip
        else:
            _lib.check(L.hb_ecc_encode(value.data_ptr(), t.data_ptr(), st[key + "::ecc"].data_ptr(), t.numel(), fmt, self._rng_mode(),
                                       self.rng_seed, int(step) & 0xFFFFFFFF, stream_id, base, stream), "hb_ecc_encode")  # fmt: skip

    @staticmethod
    def _mode_product(gemm, X, q, d: int, back: bool, out=None):
        """Contracts dimension ``d`` of X with the square matrix q: out[.., j, ..] = sum_i X[.., i, ..] q[i, j]
        (q[j, i] when ``back``). The first and last dimension are plain GEMMs on a reshaped view; a middle one is
        moved to the front first.  ``out`` (contiguous, X's shape) receives the result of a first- or last-dimension product."""
        if d == 0:
            Y = torch.empty_like(X) if out is None else out
            gemm(q, X.reshape(X.shape[0], -1), Y.view(X.shape[0], -1), ta=not back)
            return Y
        if d == X.dim() - 1:
            Y = torch.empty_like(X) if out is None else out
            gemm(X.reshape(-1, X.shape[-1]), q, Y.view(-1, X.shape[-1]), tb=back)
            return Y
        Xp = X.movedim(d, 0).contiguous()
        Y = torch.empty_like(Xp)
        gemm(q, Xp.view(Xp.shape[0], -1), Y.view(Xp.shape[0], -1), ta=not back)
        return Y.movedim(0, d).contiguous()

    @classmethod
    def _project(cls, gemm, X, Q, back: bool, out=None):
        """heavyball/utils.py:1391-1411: every dimension that has a basis is rotated by it (by its transpose when ``back``).
        The last product writes into ``out`` where it can (a first or last dimension); the caller copies otherwise."""
        dims = [d for d, q in enumerate(Q) if q is not None]
        cur = X
        for d in dims:
            direct = out is not None and d == dims[-1] and (d == 0 or d == X.dim() - 1)
            cur = cls._mode_product(gemm, cur, Q[d][0], d, back, out if direct else None)
        return cur

    @staticmethod
    def _eigh_basis(m: torch.Tensor) -> torch.Tensor:
        """Eigenvectors of the symmetric ``m`` in float64, largest eigenvalue first (heavyball/utils.py:1001-1003).  In float64: on
        a factor with a graded spectrum (singular values of the gradient spread over two decades) the vendor's fp32 eigensolver
        leaves off-diagonal terms of 1e-2 of the spectral norm in Q^T GG Q and the eigenvalues out of order, where LAPACK on the
        CPU, which the reference's fixtures come from, leaves 4e-7; in float64 it leaves 1e-15."""
        eye = torch.eye(m.shape[-1], dtype=torch.float64, device=m.device)
        _, vec = torch.linalg.eigh(m.double() + 1e-30 * eye)
        return torch.flip(vec, [-1])

    def _first_bases(self, G0, GG, fdt, seed_base: int):
        """The eigenbases of one tensor's first factors: ``_first_bases_of`` for a single entry."""
        return self._first_bases_of([(G0, GG, fdt, seed_base)])[0]

    def _first_bases_of(self, entries):
        """The eigenbases of the first factors (heavyball/utils.py:986-1038) of ``entries`` = [(G0, GG, fdt, seed_base), ...], the
        tensors (or blocks) that take their first step in this call; one list of bases per entry.

        A matrix gradient G with both factors takes one eigensolve, on its smaller side: the first factors are G G^T and G^T G,
        so the eigenvectors of one are the singular vectors of G on that side and the other side's follow as G^T U (or G U)
        with normalised columns, in the same descending order.  Where the larger factor has more columns than G has rank, the
        rest of its basis spans the null space of the factor, whose eigenvalues are rounding noise in any solver: any orthonormal
        completion is an eigenbasis to that accuracy, and a seeded random one is taken.  ``hb_orthonormalize_f32`` then makes the
        whole basis orthonormal to fp32 (its first columns already are, and stay).  An 8192-wide factor of a 2048 x 8192 gradient
        costs 37 ms this way instead of a 670 ms eigensolve.  Everything else (factors kept in 16 bits, whose stored values are
        no exact product any more; views with more than two dimensions; a single factor) takes the eigensolver per factor.

        The eigensolves of one width go to the solver as one batch: below a few thousand columns a solve is a long chain of small
        kernels, and a batch runs the chains of all its matrices side by side (twelve 768-wide factors: 27 ms instead of 216)."""
        def is_paired(G0, GG, fdt):
            return fdt == torch.float32 and G0.dim() == 2 and len(GG) == 2 and GG[0] is not None and GG[1] is not None

        wanted: Dict[tuple, List] = {}  # (device, width) -> [((entry, side), factor)]
        for e, (G0, GG, fdt, _) in enumerate(entries):
            if is_paired(G0, GG, fdt):
                sides = [0 if G0.shape[0] <= G0.shape[1] else 1]  # the smaller side
            else:
                sides = [d for d, m in enumerate(GG) if m is not None]
            for d in sides:
                wanted.setdefault((GG[d].device, GG[d].shape[-1]), []).append(((e, d), GG[d][0]))
        solved = {}
        for (_, n), lst in wanted.items():
            per = max(1, (1 << 30) // (8 * n * n))  # stacks of at most 1 GiB of float64
            for k in range(0, len(lst), per):
                part = lst[k : k + per]
                for (key, _), vec in zip(part, self._eigh_basis(torch.stack([m for _, m in part]))):
                    solved[key] = vec
        out = []
        for e, (G0, GG, fdt, seed_base) in enumerate(entries):
            Q: List[Optional[torch.Tensor]] = [None] * len(GG)
            if is_paired(G0, GG, fdt):
                s = 0 if G0.shape[0] <= G0.shape[1] else 1
                U = solved[(e, s)]
                W = (G0.T if s == 0 else G0).double() @ U  # [larger, smaller]: unnormalised singular vectors of the other side
                norms = W.norm(dim=0)
                good = norms > 1e-6 * norms.max()  # a column below that belongs to the null space of G itself
                gen = torch.Generator(device=G0.device)
                gen.manual_seed(0x50A9 + int(seed_base))  # the tensor's place in its slab: the same completion in every run
                big, small = W.shape
                other = torch.randn(big, big, device=G0.device, dtype=torch.float32, generator=gen)
                other[:, :small] = torch.where(good, (W / norms.clamp(min=1e-300)).float(), other[:, :small])
                Q[s] = U.to(fdt).contiguous()[None]
                Q[1 - s] = other[None] if orthonormalize_(other) else self._eigh_basis(GG[1 - s]).to(fdt).contiguous()
            else:
                for d, m in enumerate(GG):
                    if m is not None:
                        Q[d] = solved[(e, d)].to(fdt).contiguous()[None]
            out.append(Q)
        return out

    @staticmethod
    def _update_ggt(gemm, G, GG, a: float, one_minus_a: float):
        """heavyball/utils.py:1205-1221: GG_d <- GG_d*(1-a) + (G contracted with itself over all dimensions but d)*a."""
        for d, m in enumerate(GG):  # a vector has a factor only under precondition_1d, a scalar never
            if m is None:
                continue
            last = d == G.dim() - 1
            X = G.reshape(-1, G.shape[-1]) if last else (G if d == 0 else G.movedim(d, 0).contiguous()).reshape(G.shape[d], -1)
            depth, width = (X.shape[0], X.shape[1]) if last else (X.shape[1], X.shape[0])
            if last and depth >= 4 * _GGT_CHUNK and ((width + 127) // 128) ** 2 < 128:
                # a small factor of a very long tensor (an embedding's: 768 x 768 from 50257 rows) is a handful of tiles with
                # thousands of steps each: the rows are cut into chunks whose products are independent (they share a launch),
                # added up in chunk order and folded into the factor with the product kernel's own arithmetic,
                # m * (1 - a) + sum * a, every operation rounded once
                cuts = list(range(0, depth, _GGT_CHUNK))
                parts = torch.empty((len(cuts), width, width), dtype=torch.float32, device=G.device)
                for c, k0 in enumerate(cuts):
                    Xc = X[k0 : k0 + _GGT_CHUNK]
                    gemm(Xc, Xc, parts[c], ta=True, symmetric=True, independent=True)
                gemm.barrier()

                def fold(m=m, parts=parts):
                    total = parts.sum(dim=0)
                    total.mul_(a)
                    m[0].mul_(one_minus_a).add_(total)

                gemm.then(fold)
            elif last:
                gemm(X, X, m[0], ta=True, accumulate=True, alpha=a, beta=one_minus_a, symmetric=True)
            else:
                gemm(X, X, m[0], tb=True, accumulate=True, alpha=a, beta=one_minus_a, symmetric=True)

    def _refresh(self, gemm, jobs):
        """heavyball/utils.py:829-900 (heavy=False) for every (GG, Q, exp_avg) of ``jobs``: power-iteration step, sort by
        the estimated eigenvalues, QR, then rotate exp_avg from the old eigenbasis into the new one.

        A QR factorisation is a long chain of small dependent kernels (a 128-column panel at a time, its Cholesky factor in
        ONE workgroup), so bases of one shape are factored together (``hb_orthonormalize_f32_batched``: every launch of the
        chain covers the whole group) and the groups run side by side on streams of default priority, each started as
        soon as the ``GG @ Q`` products of its members are sorted, while the caller's stream goes on with the products
        of the other bases and, as the factorisations finish (shortest first), with the rotations that follow them.  Nothing
        is written to Q or exp_avg until every status word has come back (one copy, the only host synchronisation): a
        basis whose factor was numerically rank-deficient (early steps) is redone with Householder QR first."""
        dev = gemm.device
        main = torch.cuda.current_stream(dev)
        sides = []  # one entry per basis to refresh
        for pi, (GG, Q, exp_avg, *_) in enumerate(jobs):
            if exp_avg.dim() <= 1:  # heavyball/utils.py:837-839; a vector (bucket dimension + one) has a basis under precondition_1d
                continue
            for d, (m, q) in enumerate(zip(GG, Q)):
                if m is not None:
                    sides.append(dict(param=pi, m=m, q=q, d=d, exp_avg=exp_avg))
        if not sides:
            return
        status = torch.zeros(len(sides), dtype=torch.int32, device=dev)
        by_shape: Dict[int, List[int]] = {}  # width of the (square) basis -> its sides
        for k, sd in enumerate(sides):
            by_shape.setdefault(sd["q"][0].shape[-1], []).append(k)
        streams = self._ortho_streams(dev, len(by_shape))
        for gi, width in enumerate(sorted(by_shape, reverse=True)):  # longest chains first
            ks = by_shape[width]
            # the sides of one width together: their GG @ Q products share launches, and the estimates, their order and the
            # reordered columns are computed on stacked tensors (a model has dozens of bases of one width)
            tmp_all = torch.empty((len(ks), width, width), dtype=torch.float32, device=dev)
            gemm.defer()
            for j, k in enumerate(ks):
                gemm.owner = k
                gemm(sides[k]["m"][0], sides[k]["q"][0], tmp_all[j])
            gemm.stop()
            if len(ks) * width * width <= 1 << 26:
                eig_all = (torch.stack([sides[k]["q"][0] for k in ks]) * tmp_all).sum(dim=1)
            else:  # wide bases: no second copy of them
                eig_all = torch.stack([(sides[k]["q"][0] * tmp_all[j]).sum(dim=0) for j, k in enumerate(ks)])
            idx_all = torch.argsort(eig_all, dim=-1, descending=True, stable=True).unsqueeze(1).expand_as(tmp_all)
            ordered_all = tmp_all.gather(-1, idx_all)
            basis_all = ordered_all.clone()
            for j, k in enumerate(ks):
                sd = sides[k]
                sd["idx"], sd["ordered"], sd["basis"], sd["tmp"] = idx_all[j], ordered_all[j], basis_all[j], tmp_all[j]
                sd["job"] = _Ortho(sd["basis"], status[k : k + 1])
            # the bases of this width are sorted: their factorisations start together on the group's stream
            ready = torch.cuda.Event()
            ready.record(main)
            streams[gi].wait_event(ready)
            launch_orthonormalize([sides[k]["job"] for k in ks], streams[gi])
            done = torch.cuda.Event()
            done.record(streams[gi])
            for k in ks:
                sides[k]["done"] = done

        def finish(ks):
            """The new Q (scattered back to the old column order) of the sides ``ks`` and the rotated exp_avg of their
            parameters, all in temporaries."""
            rotated: Dict[int, torch.Tensor] = {}
            waited = None
            gemm.defer()
            for k in ks:
                sd = sides[k]
                if sd["done"] is not waited:
                    # the rotations collected so far belong to factorisations that are there: out with them, in shared launches,
                    # before the caller's stream stops for the next factorisation
                    gemm.flush()
                    main.wait_event(sd["done"])
                    waited = sd["done"]
                new_q = torch.empty_like(sd["tmp"])
                new_q.scatter_(-1, sd["idx"], sd["basis"])
                sd["new_q"] = new_q
                # back through the old basis, forward through the new one: 4 numel d FLOP, where an explicit change of
                # basis Q^T Q_new would cost 2 d^3 + 2 numel d (the order an einsum planner picks for the reference's
                # five-operand expression, heavyball/utils.py:877-884, as well)
                E = rotated.get(sd["param"], sd["exp_avg"][0])
                if E.dim() > 2:  # a middle dimension is moved to the front by a copy, which must see the product before it
                    gemm.stop()
                gemm.owner = sd["param"]
                E = self._mode_product(gemm, E, sd["q"][0], sd["d"], back=True)
                E = self._mode_product(gemm, E, new_q, sd["d"], back=False)
                rotated[sd["param"]] = E
                if gemm.queue is None:
                    gemm.defer()
            gemm.stop()
            return rotated

        # optimistic pass: parameters whose longest factorisation is shortest first; the rotations of one parameter in
        # dimension order (as the reference applies them)
        longest: Dict[int, int] = {}
        for sd in sides:
            longest[sd["param"]] = max(longest.get(sd["param"], 0), sd["q"][0].numel())
        seq = sorted(range(len(sides)), key=lambda k: (longest[sides[k]["param"]], sides[k]["param"], sides[k]["d"]))
        rotated = finish(seq)
        ok = (status.cpu() == 0).tolist()
        if not all(ok):
            bad_params = {sides[k]["param"] for k in range(len(sides)) if not ok[k]}
            redo = [k for k in seq if sides[k]["param"] in bad_params]
            for k in redo:
                if not ok[k]:  # rank-deficient factor: Householder QR copes with that
                    sides[k]["basis"] = torch.linalg.qr(sides[k]["ordered"]).Q
            rotated.update(finish(redo))
        for pi, E in rotated.items():
            jobs[pi][2][0].copy_(E)
        for sd in sides:
            sd["q"][0].copy_(sd["new_q"])

    #: let the products of different tensors share launches (hb_gemm_f32_grouped); False runs every tensor on its own, one product
    #: after the other, which tests use to compare the two routes
    group_products = True

    def _ortho_streams(self, dev, n: int):
        pool = self.__dict__.setdefault("_side_streams", {}).setdefault(dev, [])
        while len(pool) < n:
            pool.append(torch.cuda.Stream(device=dev))  # default priority
        return pool[:n]

"""SOAP, CPU restatement (test infrastructure; see oracle/__init__.py).

Follows heavyball/chainable.py:1235-1275 (``_init_soap``, ``_apply_soap_preconditioner``, ``scale_by_soap``),
heavyball/utils.py:1205-1221 (``update_ggt``), :1362-1388 (``init_preconditioner``), :1391-1411 (``project``),
:829-900 (``get_orthogonal_matrix_QR``), :986-1038 (``_stable_symmetric_basis``, ``get_orthogonal_matrix``),
:1852-1883 (``adam_``), :3494-3500 (``psgd_should_update``) and heavyball/__init__.py:839-909 (``SOAP`` defaults).

State tensors carry the leading bucket dimension of the reference (heavyball/chainable.py:550-552); every parameter
is its own bucket here (n = 1), which is also what the reference does for parameters of distinct shapes.
"""

from typing import List, Optional

import numpy as np

import torch
from torch import Tensor

from .first_order import beta_debias, f32, ieee_sqrt, step_lr, update_param_

einsum_base = "abcdefghijklmnopqrstuvwxyz"


def should_update(group: dict, prob: float, name="cumulative_prob") -> bool:
    """heavyball/utils.py:3494-3500: fires when the float-accumulated probability crosses an integer."""
    group[f"{name}_prob_step"] = group.get(f"{name}_prob_step", 0) + 1
    cumulative = group.get(name, 0)
    group[name] = cumulative + prob
    return int(group[name]) > int(cumulative)


def merged_shape(shape, max_precond_dim: int):
    """heavyball/utils.py:240-272 (``dim_merger`` with split=False), applied to every parameter and gradient when the group
    has merge_dims (heavyball/utils.py:3726-3742, :1612-1623): trailing dimensions are merged from the right while the
    product stays <= max_precond_dim; the leading dimension is never merged into."""
    if len(shape) == 0:
        return []
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
    return [shape[0], *new_shape[::-1]]


def dim_merger(t: Tensor, max_precond_dim: int, split: bool):
    """heavyball/utils.py:240-286 on a tensor: the merged view; with ``split`` every dimension larger than max_precond_dim is
    cut into blocks of at most that size (the blocks of the last such dimension outermost in the order), dimensions of size
    one are dropped from the blocks, and each block is merged again.  A tensor that needs no cut comes back as the merged view."""
    new = t.reshape(merged_shape(t.shape, max_precond_dim))
    if not split:
        return new
    blocks = [new]
    for i, sh in reversed(list(enumerate(new.shape))):
        if sh == 1:
            blocks = [b.squeeze(dim=i) for b in blocks]
            continue
        if sh <= max_precond_dim:
            continue
        blocks = [a for b in blocks for a in b.split(max_precond_dim, dim=i)]
    if len(blocks) == 1:
        return new
    out = []
    for b in blocks:
        r = dim_merger(b, max_precond_dim, split)
        if isinstance(r, list):
            out.extend(r)
        else:
            out.append(r)
    return out


def side_noise_index(tidx, n: int):
    """The tensor index handed to the rounding for a factor or a basis of n elements that belongs to (the block of) a parameter:
    element e takes the noise of place ``start + e`` of the parameter, ``start`` being where the block's own moments start."""
    if isinstance(tidx, tuple):
        return (tidx[0], np.uint64(tidx[1][0] if len(tidx[1]) else 0) + np.arange(n, dtype=np.uint64))
    return (tidx, np.arange(n, dtype=np.uint64))


def update_ggt(grad: Tensor, GG: List[Optional[Tensor]], max_precond_dim: int, precondition_1d: bool, beta, rounding=None, tidx=0):
    """heavyball/utils.py:1205-1221: GG_i <- GG_i * (1 - a) + (contraction of grad with itself over all but dim i) * a, a = 1 - beta.
    A factor kept in a 16-bit dtype (it has the dtype of the gradient it was created from, :1381) is rewritten through
    copy_stochastic_ (:1048); the contraction runs in the dtype of ``grad`` as handed over: the gradient's own on the first step
    (:1387), fp32 afterwards (heavyball/chainable.py:1248)."""
    from . import first_order as fo
    from . import philox
    from .rounding import HalfRounding

    if grad.dim() == 2 and (not precondition_1d or grad.shape[1] > max_precond_dim):
        return
    g0 = einsum_base[: grad.dim() - 1]
    for idx, m in enumerate(GG):
        if not isinstance(m, Tensor):
            continue
        b = einsum_base[idx]
        g1 = g0.replace(b, b.upper())
        outer = torch.einsum(f"...{g0},...{g1}->...{b + b.upper()}", grad, grad)
        a = 1 - beta
        a = a.to(torch.float32) if isinstance(a, Tensor) else f32(a)
        if m.dtype == torch.float32:
            m.copy_(m * (1 - a) + outer * a)  # stochastic_lerp_ on fp32 (heavyball/utils.py:1048)
        else:
            fo.copy_stochastic(m, fo.promote(m) * (1 - a) + fo.promote(outer) * a, rounding or HalfRounding(), philox.STREAM_SOAP_GG + 2 * idx,
                               side_noise_index(tidx, m.numel()))  # fmt: skip


def symmetric_basis(m: Tensor, min_eps=1e-30) -> Tensor:
    """heavyball/utils.py:986-1003 on the path that does not raise: eigh(m + eps I), eigenvectors in descending order."""
    from . import first_order as fo

    m32 = fo.promote(m)  # :992; the basis goes back to the factor's dtype (:996, :1003)
    eye = torch.eye(m32.shape[-1], dtype=m32.dtype)
    _, vec = torch.linalg.eigh(m32 + min_eps * eye)
    return torch.flip(vec, [-1]).contiguous().to(m.dtype)


def init_preconditioner(grad: Tensor, max_precond_dim: int, precondition_1d: bool, rounding=None, tidx=0):
    """heavyball/utils.py:1362-1388 with init_factor = 0; ``grad`` carries the bucket dimension.  Factors and bases take the
    gradient's dtype."""
    GG: List[Optional[Tensor]] = []
    if grad.numel() > 1 and (grad.ndim > 2 or precondition_1d):
        n = grad.shape[0]
        for sh in grad.shape[1:]:
            if sh > max_precond_dim or sh == 1:
                GG.append(None)
            else:
                GG.append(torch.zeros(n, sh, sh, dtype=grad.dtype))
    else:
        GG.append(None)
    update_ggt(grad, GG, max_precond_dim, precondition_1d, 0, rounding, tidx)
    Q = [None if m is None else symmetric_basis(m) for m in GG]
    return GG, Q


def project(grad: Tensor, Q: List[Optional[Tensor]], back: bool) -> Tensor:
    """heavyball/utils.py:1391-1411."""
    param = einsum_base[: grad.dim() - 1]
    pre = ",".join(["..." + (g + g.upper())[:: -1 if back else 1] for m, g in zip(Q, param) if m is not None])
    if pre:
        out = "".join([c.upper() if c.upper() in pre else c for c in param])
        from . import first_order as fo

        grad = torch.einsum(f"...{param},{pre}->...{out}", fo.promote(grad), *[fo.promote(q) for q in Q if q is not None]).to(grad.dtype)
    return grad


def adam_(exp_avg, exp_avg_sq, grad: Tensor, beta1, beta2, step: Tensor, eps, rounding=None, tidx=0) -> Tensor:
    """heavyball/utils.py:1852-1883: returns exp_avg / max(sqrt(exp_avg_sq), eps) from the moments as computed in fp32, BEFORE
    they are written back to their storage (fp32: the same values; bf16 or an ECC pair: rounded on the way, :1842-1849)."""
    from . import first_order as fo
    from . import philox
    from .rounding import HalfRounding

    rounding = rounding or HalfRounding()
    beta1, beta2, eps = f32(beta1), f32(beta2), f32(eps)
    b1 = beta_debias(beta1, step)
    b2 = beta_debias(beta2, step)
    exp_avg32 = fo.lerp_([exp_avg], [grad], b1, rounding, philox.STREAM_EXP_AVG, [tidx])[0]
    denom = fo.exp_avg_sq_([exp_avg_sq], [grad], b2, eps, rounding, [tidx])[0]
    return exp_avg32 / denom


def refresh_basis(GG: List[Optional[Tensor]], Q: List[Optional[Tensor]], exp_avg, rounding=None, tidx=0):
    """heavyball/utils.py:829-900 (heavy=False): one power-iteration step + QR per side, then rotate exp_avg into the new basis
    (decoded to fp32 for the rotation and written back through copy_stochastic_, :883-884).

    Returns the smallest gap between two neighbouring sort keys (the estimates ``diag(Q^T GG Q)`` that order the columns, :871-873)
    relative to the largest one, over all sides; 1.0 when nothing was sorted.  The order of two keys that agree to fp32 rounding
    is decided by the summation order of the products, so a checker can tell from this figure when the column order - and with it
    the rotated exp_avg - is not determined by the data."""
    from . import first_order as fo
    from . import philox
    from .rounding import HalfRounding

    stored = exp_avg
    exp_avg = fo.promote(stored)
    if exp_avg.dim() <= 1:
        return 1.0
    new_qs = []
    key_gap = 1.0
    for m, q in zip(GG, Q):
        if m is None:
            new_qs.append(None)
            continue
        m, q = fo.promote(m), fo.promote(q)  # heavyball/utils.py:850, :857
        tmp = m @ q
        eig = torch.einsum("...ij,...ij->...j", q, tmp)
        if eig.shape[-1] > 1:
            keys = eig.double().sort(dim=-1, descending=True).values
            key_gap = min(key_gap, ((keys[..., :-1] - keys[..., 1:]).min() / keys.abs().max().clamp_min(1e-300)).item())
        idx = torch.argsort(eig, descending=True).unsqueeze(-2).expand_as(tmp)
        tmp.scatter_(-1, idx, torch.linalg.qr(tmp.gather(-1, idx)).Q)
        new_qs.append(tmp)
    pd = exp_avg.dim() - 1
    in_str, out_str = einsum_base[:pd], einsum_base[pd : 2 * pd]
    from_sh = ",".join([f"...{o}{i}" for m, i, o in zip(Q, in_str, in_str.upper()) if m is not None])
    if not from_sh:
        return key_gap
    to_sh = ",".join([f"...{i}{o}" for m, i, o in zip(new_qs, in_str.upper(), out_str) if m is not None])
    out_lin = "".join([o if o in to_sh else i for i, o in zip(in_str, out_str)])
    subs = f"...{in_str},{from_sh},{to_sh}->...{out_lin}"
    rotated = torch.einsum(subs, exp_avg, *[fo.promote(q) for q in Q if q is not None], *[q for q in new_qs if q is not None])
    fo.copy_stochastic(stored, rotated, rounding or HalfRounding(), philox.STREAM_SOAP_ROTATE, tidx)
    for li, (q, qn) in enumerate(zip(Q, new_qs)):
        if q is None:
            continue
        if q.dtype == torch.float32:
            q.copy_(qn)
        else:  # heavyball/utils.py:898-900: the new basis into a 16-bit one through copy_stochastic_
            fo.copy_stochastic(q, qn, rounding or HalfRounding(), philox.STREAM_SOAP_Q + 2 * li, side_noise_index(tidx, q.numel()))
    return key_gap


class SOAPOracle:
    """heavyball.SOAP (heavyball/__init__.py:861-909).  With ``split`` a parameter larger than max_precond_dim in some dimension is
    preconditioned block by block (heavyball/utils.py:274-286, :1612-1623): every block has its own state, ``state[i]`` holding
    that of block 0 and ``block_state[i][k]`` that of block k >= 1."""

    def __init__(self, params, lr=3e-3, betas=(0.9, 0.95), shampoo_beta=0.95, eps=1e-8, weight_decay=0.01, precondition_frequency=2,
                 max_precond_dim=2048, precondition_1d=False, warmup_steps=0, gradient_clipping=None,
                 update_clipping=None, mars=False, mars_gamma=0.0025, ecc=None, storage_dtype="float32", param_ecc=None,
                 caution=False, cautious_weight_decay=False, precond_grad_accum=False, palm=False, beta2_scale=0.8, merge_dims=True,
                 split=False, rounding=None):  # fmt: skip
        from . import philox
        from .ecc import MODES, EccTensor
        from .rounding import HalfRounding

        # precond_grad_accum is read by PSGD's guard only (heavyball/chainable.py:304-345): SOAP's chain ignores it
        self.rounding = rounding or HalfRounding()
        self.ecc, self.storage_dtype = ecc, getattr(torch, storage_dtype)
        self.caution, self.cautious_weight_decay = caution, cautious_weight_decay
        self.param_ecc = param_ecc
        self.mars, self.mars_gamma = mars, mars_gamma
        self.palm, self.beta2_scale, self.merge_dims = palm, beta2_scale, merge_dims
        self.split = split and merge_dims  # heavyball/utils.py:3726-3728: without merge_dims nothing is merged or cut
        self.max_precond_dim = max_precond_dim
        self.block_state = [dict() for _ in params]
        self._state_init = [dict() for _ in params]
        if param_ecc is not None:  # heavyball/chainable.py:2421-2444: the live parameter is narrowed at construction
            narrowed = []
            for i, p in enumerate(params):
                pd, cd = MODES[param_ecc]
                e = EccTensor(p.to(pd), torch.zeros(p.shape, dtype=cd))
                if p.dtype != pd:
                    e.compute_correction(p.float(), self.rounding.at_step(0).uniform(philox.STREAM_INIT_PARAM, i, p.shape))
                narrowed.append(e)
                # heavyball/chainable.py:2438-2444: one correction tensor per view of the parameter, i.e. per block under split
                for k, blk in enumerate(self._views(e)):
                    (self._state_init[i] if k == 0 else self.block_state[i].setdefault(k, {}))["param::ecc"] = blk.corr
            params = narrowed
        self.params = params
        self.gradient_clipping, self.update_clipping = gradient_clipping, update_clipping
        self.lr, self.betas, self.shampoo_beta, self.eps = lr, betas, shampoo_beta, eps
        self.weight_decay, self.max_precond_dim, self.precondition_1d = weight_decay, max_precond_dim, precondition_1d
        self.warmup_steps = warmup_steps
        self.schedule = 1 / precondition_frequency
        self.inner_group = {}
        self.state = self._state_init
        self.step_count = torch.zeros((), dtype=torch.int64)
        self.fired = []
        self.sort_key_gap = {}  # (tensor, block) -> smallest relative gap of the sort keys over the refreshes so far

    def _moment(self, st, key, like):
        """zero_guard with the group's storage (heavyball/chainable.py:277-301)."""
        from .ecc import EccTensor

        if key not in st:
            if self.ecc is None:
                st[key] = torch.zeros_like(like, dtype=self.storage_dtype)
            else:
                e = EccTensor.zeros(like.shape, self.ecc)
                st[key], st[key + "::ecc"] = e.primary, e.corr
        return st[key] if self.ecc is None else EccTensor(st[key], st[key + "::ecc"])

    K_OLD = "mars_mars_old_grad_5"  # pinned by a trajectory written from the reference
    K_M, K_V, K_Q, K_GG = "scale_by_soap_exp_avg_2", "scale_by_soap_exp_avg_sq_2", "scale_by_soap_Q_3", "scale_by_soap_GG_3"

    def _views(self, t):
        """The views the chain runs on (heavyball/utils.py:1612-1623): the blocks of a split tensor or ECC pair, cut alike; the
        tensor itself otherwise."""
        from .ecc import EccTensor

        if not self.split:
            return [t]
        if isinstance(t, EccTensor):
            return [EccTensor(a, b) for a, b in zip(self._views(t.primary), self._views(t.corr))]
        r = dim_merger(t, self.max_precond_dim, True)
        return r if isinstance(r, list) else [t]

    def _block_state(self, i, k):
        return self.state[i] if k == 0 else self.block_state[i].setdefault(k, {})

    def _noise_index(self, i, shape, private=False):
        """What the rounding is handed as the tensor index of the blocks of parameter i.  Without split: i.  With split, per block,
        (i, offsets): state that lives in the parameter's own layout (the parameter, its correction, MARS' old gradient) takes the
        noise of the elements' places in the parameter; the moments of the preconditioner, one tensor per block, take consecutive
        runs (``private``)."""
        if not self.split:
            return [i]
        idx = self._views(torch.arange(int(np.prod(shape)) if len(shape) else 1).reshape(shape))
        if not private:
            return [(i, b.reshape(-1).numpy().astype(np.uint64)) for b in idx]
        out, start = [], 0
        for b in idx:
            out.append((i, np.arange(start, start + b.numel(), dtype=np.uint64)))
            start += b.numel()
        return out

    def _view_shape(self, shape):
        """heavyball/utils.py:3726-3742: without merge_dims the tensors are taken as they are."""
        return merged_shape(shape, self.max_precond_dim) if self.merge_dims else list(shape)

    def step(self, grads):
        is_precond = should_update(self.inner_group, self.schedule)
        self.step_count = self.step_count + 1
        step = self.step_count
        if self.palm:  # heads the chain (heavyball/chainable.py:2693-2694) and rewrites the group's betas
            from . import first_order as fo

            self.betas = fo.palm_betas(self.betas, step, self.beta2_scale)
        self.fired.append(bool(is_precond))
        lr = step_lr(self.lr, step, self.warmup_steps)
        todo_p, todo_u, todo_g, todo_i = [], [], [], []
        updates = {i: g.clone() for i, g in enumerate(grads) if g is not None}
        if self.mars and updates:  # heavyball/chainable.py:642-647 heads the chain; the gradient becomes the corrected one
            from . import first_order as fo

            keys = list(updates)
            # zero_guard with the group's storage, like the moments (heavyball/chainable.py:277-301), in the shape of the view the
            # chain runs on: the parameter's own, or a block's under split (the blocks are views: the correction lands in updates[k])
            ub, ob, tb = [], [], []
            for k in keys:
                for bk, (u, t) in enumerate(zip(self._views(updates[k]), self._noise_index(k, updates[k].shape))):
                    ub.append(u)
                    ob.append(self._moment(self._block_state(k, bk), self.K_OLD, u))
                    tb.append(t)
            fo.mars_correction(ub, ob, self.mars_gamma, self.betas[0], self.rounding.at_step(int(step)), tb)
            grads = [updates[i].clone() if i in updates else None for i in range(len(grads))]
        if self.gradient_clipping is not None and updates:  # heavyball/chainable.py:2696-2699: on the update, ahead of the transform
            from . import first_order as fo

            fn = {"l2_clip_": fo.l2_clip, "rmsnorm_clip_": fo.rmsnorm_clip, "global_l2norm_clip": fo.global_l2norm_clip,
                  "global_rmsnorm_clip": fo.global_rmsnorm_clip}[self.gradient_clipping]  # fmt: skip
            from . import philox

            views, tix = [], []  # under split the norms are per block
            for k in updates:
                views += self._views(updates[k])
                tix += self._noise_index(k, updates[k].shape)
            for u, c, t in zip(views, fn(views), tix):  # heavyball/utils.py:3226-3232 writes back through copy_stochastic_
                fo.copy_stochastic(u, c, self.rounding.at_step(int(step)), philox.STREAM_CLIP, t)
        for i, (p, g) in enumerate(zip(self.params, grads)):
            if g is None:
                continue
            # blocks of the parameter, of the gradient and of the update, cut alike
            blocks = list(zip(self._views(p), self._views(g), self._views(updates[i])))
            private = self._noise_index(i, g.shape, private=True)
            shared = self._noise_index(i, g.shape)
            for k, (p, g, upd) in enumerate(blocks):
                st = self._block_state(i, k)
                from . import first_order as fo

                # merged view + the bucket dimension; the preconditioner promotes what it is handed (heavyball/chainable.py:1261, :1248)
                u = fo.promote(upd).reshape(self._view_shape(g.shape)).unsqueeze(0)
                rounding = self.rounding.at_step(int(step))
                if self.K_M not in st:  # first step: ZeroGuard + GeneralGuard init, no update (heavyball/chainable.py:372-377)
                    self._moment(st, self.K_M, u)
                    self._moment(st, self.K_V, u)
                    # heavyball/chainable.py:1235-1238: the initial factors come from the gradient, not from the (clipped) update
                    g0 = g.clone().reshape(self._view_shape(g.shape)).unsqueeze(0)
                    st[self.K_GG], st[self.K_Q] = init_preconditioner(g0, self.max_precond_dim, self.precondition_1d, rounding, private[k])
                    continue
                Q, GG = st[self.K_Q], st[self.K_GG]
                gp = project(u, Q, False)
                m_st, v_st = self._moment(st, self.K_M, u), self._moment(st, self.K_V, u)
                precond = adam_(m_st, v_st, gp, self.betas[0], self.betas[1], step - 1, self.eps, rounding, private[k])
                precond = project(precond, Q, True)
                beta = beta_debias(self.shampoo_beta, step)  # heavyball/chainable.py:1244
                update_ggt(u, GG, self.max_precond_dim, self.precondition_1d, beta, rounding, private[k])
                if is_precond:
                    gap = refresh_basis(GG, Q, m_st, rounding, private[k])
                    self.sort_key_gap[(i, k)] = min(self.sort_key_gap.get((i, k), 1.0), gap)
                todo_p.append(p)
                todo_u.append(precond.squeeze(0).reshape(p.shape))
                todo_g.append(g)
                todo_i.append(shared[k])
        if todo_p and self.update_clipping is not None:  # heavyball/chainable.py:2700-2701
            from . import first_order as fo

            fn = {"l2_clip_": fo.l2_clip, "rmsnorm_clip_": fo.rmsnorm_clip, "global_l2norm_clip": fo.global_l2norm_clip,
                  "global_rmsnorm_clip": fo.global_rmsnorm_clip}[self.update_clipping]  # fmt: skip
            todo_u = fn(todo_u)
        if todo_p:
            update_param_(todo_p, todo_u, lr, self.weight_decay, self.caution, self.cautious_weight_decay, todo_g,
                          self.rounding.at_step(int(step)), todo_i)

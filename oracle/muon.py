"""Muon: Nesterov-EMA momentum and Newton-Schulz orthogonalisation, CPU restatement (test infrastructure; see
oracle/__init__.py).

Follows heavyball/utils.py:766-769 (``_compilable_nesterov_ema_``), :550-577 (``zeropower_via_newtonschulz5``),
:637-657 (``legacy_zeropower_via_newtonschulz5``), :605-631 (``msign``), :784-817 (``_compilable_orthogonal_``: which schedule runs and the
``max(1, rows/cols) ** 0.5`` post-scale) and heavyball/chainable.py:1117-1138 (``orthogonalize_update``, ``nesterov_ema``).

bf16 matrix products call the same ATen op as the reference (``@`` on bf16 tensors): an fp32-accumulated product rounded
once to bf16, up to the order of the accumulation, which no two backends share (on 64x64 inputs a plain fp32 matmul of
the same operands, rounded to bf16, already ends 5e-3 away after five iterations); parity of the Newton-Schulz output is
therefore a tolerance (2e-2 relative Frobenius), not bit equality.  PARITY OF THE
NEWTON-SCHULZ NUMERICS IS NOT PINNED BY ANY TEST OF THE REFERENCE (none calls zeropower_*); it is pinned here by golden
vectors written from the reference (tests/golden/ns5.pt; ns5_bf16.pt and ns5_fp16.pt for 16-bit update buffers; msign.pt for the
ten-step schedule) and by the polar-factor invariant.
"""

from typing import List

import torch
from torch import Tensor

from . import philox
from .ecc import EccTensor, copy_stochastic, promote, stochastic_round
from .first_order import beta_debias, f32, lerp_, step_lr, update_param_
from .rounding import HalfRounding

NS_COEFFS = (  # heavyball/utils.py:561-567
    (4.0848, -6.8946, 2.9270),
    (3.9505, -6.3029, 2.6377),
    (3.7418, -5.5913, 2.3037),
    (2.8769, -3.1427, 1.2046),
    (2.8366, -3.0525, 1.2012),
)
LEGACY_COEFFS = ((3.4445, -4.7750, 2.0315),) * 5  # heavyball/utils.py:639
# heavyball/utils.py:587-602, :619: the published polynomials of arXiv 2505.16932v3, all but the last divided by a safety factor
# (a / 1.01, b / 1.01^3, c / 1.01^5); a schedule longer than the table repeats its last entry.
_POLAR = (
    (8.28721201814563, -23.595886519098837, 17.300387312530933),
    (4.107059111542203, -2.9478499167379106, 0.5448431082926601),
    (3.9486908534822946, -2.908902115962949, 0.5518191394370137),
    (3.3184196573706015, -2.488488024314874, 0.51004894012372),
    (2.300652019954817, -1.6689039845747493, 0.4188073119525673),
    (1.891301407787398, -1.2679958271945868, 0.37680408948524835),
    (1.8750014808534479, -1.2500016453999487, 0.3750001645474248),
    (1.875, -1.25, 0.375),
)
_POLAR_STABLE = tuple((a / 1.01, b / 1.01**3, c / 1.01**5) for a, b, c in _POLAR[:-1]) + (_POLAR[-1],)
POLAR_COEFFS = tuple(_POLAR_STABLE[min(k, len(_POLAR_STABLE) - 1)] for k in range(10))  # msign(x, 10), heavyball/utils.py:796-797


def bf16_matmul(a: Tensor, b: Tensor) -> Tensor:
    """The reference's own op: ``@`` on bf16 tensors (heavyball/utils.py:568-573).  ATen's CPU kernel accumulates in
    fp32 and rounds once to bf16, in a blocking of its own choosing."""
    return a @ b


def _iterate(x: Tensor, coeffs) -> Tensor:
    """heavyball/utils.py:568-573: s = x x^T; y = c s + b I; y = y s + a I; x = y x, every intermediate in bf16."""
    for a, b, c in coeffs:
        s = bf16_matmul(x, x.mT)
        y = c * s
        y.diagonal(dim1=-2, dim2=-1).add_(b)
        y = bf16_matmul(y, s)
        y.diagonal(dim1=-2, dim2=-1).add_(a)
        x = bf16_matmul(y, x)
    return x


def newton_schulz5(G: Tensor, noise16: Tensor, eps=1e-7) -> Tensor:
    """heavyball/utils.py:550-577 for fp32 input; ``noise16`` replaces the draw of the bf16 stochastic rounding (:556)."""
    Gn = G / G.norm(dim=(-2, -1)).clamp(min=eps)
    x = stochastic_round(Gn, noise16)
    if G.size(-2) > G.size(-1):
        x = x.mT
    x = _iterate(x, NS_COEFFS)
    if G.size(-2) > G.size(-1):
        x = x.mT
    return x.to(G.dtype)


def polar_express(G: Tensor, noise16: Tensor, eps=1e-7) -> Tensor:
    """heavyball/utils.py:605-631 (``msign`` with steps = 10): normalisation, input rounding and iteration of newton_schulz5 under
    the ten-step schedule above."""
    Gn = G / G.norm(dim=(-2, -1)).clamp(min=eps)
    x = stochastic_round(Gn, noise16)
    if G.size(-2) > G.size(-1):
        x = x.mT
    x = _iterate(x, POLAR_COEFFS)
    if G.size(-2) > G.size(-1):
        x = x.mT
    return x.to(G.dtype)


def legacy_newton_schulz5(G: Tensor, noise16_a: Tensor, noise16_b: Tensor, eps=1e-7) -> Tensor:
    """heavyball/utils.py:637-657: round to bf16 first, then divide by max(norm, eps) (a second stochastic round)."""
    x = stochastic_round(G.clone(), noise16_a)
    x = stochastic_round(x.float() / G.norm(dim=(-2, -1)).clamp(min=f32(eps)), noise16_b)
    if G.size(0) > G.size(1):
        x = x.T
    x = _iterate(x, LEGACY_COEFFS)
    if G.size(0) > G.size(1):
        x = x.T
    return x.to(G.dtype)


def orthogonal(x: Tensor, rounding, tidx: int, mode="newtonschulz") -> Tensor:
    """heavyball/utils.py:784-817 with scale_mode="scale": non-square inputs always take the per-iteration schedule."""
    if mode == "newtonschulz" or x.shape[-2] != x.shape[-1]:
        y = newton_schulz5(x, rounding.noise16(philox.STREAM_NS_INPUT, tidx, x.shape))
    elif mode == "thinky_polar_express":
        y = polar_express(x, rounding.noise16(philox.STREAM_NS_INPUT, tidx, x.shape))
    elif mode == "legacy_newtonschulz":
        y = legacy_newton_schulz5(x, rounding.noise16(philox.STREAM_NS_INPUT, tidx, x.shape), rounding.noise16(philox.STREAM_NS_INPUT + 1, tidx, x.shape))
    else:
        raise NotImplementedError(mode)
    y *= max(1, x.size(-2) / x.size(-1)) ** 0.5
    return y


def nesterov_ema_(state: List[Tensor], grad: List[Tensor], beta, rounding, tidx):
    """heavyball/utils.py:766-769: m <- lerp(m, g, beta) (no debias); g <- g + m."""
    beta = f32(beta)
    ema32 = lerp_(state, grad, beta, rounding, philox.STREAM_EXP_AVG, tidx)
    for g_, e_, t in zip(grad, ema32, tidx):
        copy_stochastic(g_, promote(g_) + e_ * 1, rounding, philox.STREAM_MARS_SR, t)


def exp_avg_(state: List[Tensor], grad: List[Tensor], beta, rounding, tidx):
    """heavyball/chainable.py:652-653 + heavyball/utils.py:457-467: m <- lerp(m, g, beta') with the debiased beta; g <- m."""
    beta = f32(beta)
    ema32 = lerp_(state, grad, beta, rounding, philox.STREAM_EXP_AVG, tidx)
    for g_, e_, t in zip(grad, ema32, tidx):
        copy_stochastic(g_, e_, rounding, philox.STREAM_MARS_SR, t)


def heavyball_momentum_(state: List[Tensor], grad: List[Tensor], beta, rounding, tidx, nesterov: bool):
    """heavyball/utils.py:737-749: v = m*beta + g; m <- v; g <- v (heavy ball) or g + v*beta (Nesterov)."""
    beta = f32(beta)
    for s_, g_, t in zip(state, grad, tidx):
        v = promote(s_) * beta + promote(g_)
        copy_stochastic(s_, v, rounding, philox.STREAM_EXP_AVG, t)
        copy_stochastic(g_, promote(g_) + v * beta if nesterov else v, rounding, philox.STREAM_MARS_SR, t)


class MuonOracle:
    """heavyball.Muon (heavyball/__init__.py:684-737); the momentum form follows ``nesterov`` / ``heavyball_momentum``
    as at :723-729, the state name the transform that owns it (heavyball/chainable.py:73-74)."""

    def __init__(self, params, lr=0.0025, betas=(0.9, 0.99), weight_decay=0.0, warmup_steps=0, caution=False,
                 cautious_weight_decay=False, rounding=None, mode="newtonschulz", nesterov=True, heavyball_momentum=False,
                 gradient_clipping=None, update_clipping=None, ecc=None, storage_dtype="float32", mars=False, mars_gamma=0.0025,
                 param_ecc=None):  # fmt: skip
        from .first_order import narrow_params

        self.rounding = rounding or HalfRounding()
        self.params = narrow_params(params, param_ecc, self.rounding)
        self.mars, self.mars_gamma = mars, mars_gamma
        self.ecc, self.storage_dtype = ecc, getattr(torch, storage_dtype)
        self.gradient_clipping, self.update_clipping = gradient_clipping, update_clipping
        self.nesterov, self.heavyball_momentum = nesterov, heavyball_momentum
        if heavyball_momentum:
            self.KEY = "nesterov_momentum_momentum_2" if nesterov else "heavyball_momentum_momentum_2"
        elif not nesterov:
            self.KEY = "exp_avg_exp_avg_2"
        self.lr, self.betas, self.weight_decay, self.warmup_steps = lr, betas, weight_decay, warmup_steps
        self.caution, self.cautious_weight_decay = caution, cautious_weight_decay
        self.mode = mode
        self.state = [dict() for _ in params]
        for i, e in enumerate(self.params):
            if isinstance(e, EccTensor):
                self.state[i]["param::ecc"] = e.corr
        self.step_count = torch.zeros((), dtype=torch.int64)

    KEY = "nesterov_ema_momentum_2"

    @property
    def MARS_KEY(self):
        """MARS' guard comes two places behind the momentum's in the reference's index walk (heavyball/chainable.py:2347-2382):
        mars_mars_old_grad_4 for Muon, _6 for MuonAdamW (pinned by trajectories written from the reference)."""
        return f"mars_mars_old_grad_{int(self.KEY.rsplit('_', 1)[1]) + 2}"

    def _guarded(self, i, key):
        """zero_guard with the group's storage (heavyball/chainable.py:277-301): plain or an ECC pair."""
        st = self.state[i]
        if key not in st:
            if self.ecc is None:
                st[key] = torch.zeros(tuple(self.params[i].shape), dtype=self.storage_dtype)
            else:
                e = EccTensor.zeros(self.params[i].shape, self.ecc)
                st[key], st[key + "::ecc"] = e.primary, e.corr
        return st[key] if self.ecc is None else EccTensor(st[key], st[key + "::ecc"])

    def step(self, grads):
        from . import first_order as fo

        fo.run_clip_points([self.step_gen(grads)])

    def step_gen(self, grads):
        """The step as a generator that yields ``(clip kind, tensors)`` where the chain clips (heavyball/chainable.py:2696-2701) and is
        sent the clipped tensors back: a group with two routes (MuonAdamW) clips the tensors of both at once."""
        idx = [i for i, g in enumerate(grads) if g is not None]
        if not idx:
            return
        self.step_count = self.step_count + 1
        step = self.step_count
        lr = step_lr(self.lr, step, self.warmup_steps)
        rounding = self.rounding.at_step(int(step))
        p = [self.params[i] for i in idx]
        grad = [grads[i] for i in idx]
        update = [g.clone() for g in grad]
        if self.mars:  # heavyball/chainable.py:2698-2699, :642-647: first in the chain; the gradient becomes the corrected one
            from . import first_order as fo

            old = [self._guarded(i, self.MARS_KEY) for i in idx]
            fo.mars_correction(update, old, self.mars_gamma, self.betas[0], rounding, idx)
            for g_, u_ in zip(grad, update):
                g_.copy_(u_)
        if self.gradient_clipping is not None:  # heavyball/chainable.py:2696-2699: on the update, ahead of the momentum
            clipped = yield (self.gradient_clipping, update, idx)
            for j, (u, c) in enumerate(zip(update, clipped)):
                if u.dtype == torch.bfloat16:
                    u.copy_(stochastic_round(c, rounding.noise16(philox.STREAM_CLIP, idx[j], u.shape)))
                else:
                    u.copy_(c.to(u.dtype))
        mom = [self._guarded(i, self.KEY) for i in idx]
        if self.heavyball_momentum:
            heavyball_momentum_(mom, update, self.betas[0], rounding, idx, self.nesterov)
        elif self.nesterov:
            nesterov_ema_(mom, update, self.betas[0], rounding, idx)
        else:
            exp_avg_(mom, update, beta_debias(self.betas[0], step), rounding, idx)  # heavyball/chainable.py:653
        out = []
        for u, i in zip(update, idx):  # heavyball/chainable.py:1117-1126
            if u.dim() < 2:
                out.append(u)
                continue
            shape = u.shape
            out.append(orthogonal(u.flatten(1, -1), rounding, i, self.mode).reshape(shape))
        if self.update_clipping is not None:  # heavyball/chainable.py:2700-2701
            clipped = yield (self.update_clipping, out, idx)
            # heavyball/utils.py:3226-3232: written back into the update buffer, which has the gradient's dtype (a stochastic
            # round into bfloat16, a plain copy otherwise)
            out = [stochastic_round(c, rounding.noise16(philox.STREAM_UPDATE_CLIP, t, o.shape)) if o.dtype == torch.bfloat16 else c.to(o.dtype)
                   for o, c, t in zip(out, clipped, idx)]  # fmt: skip
        update_param_(p, out, lr, self.weight_decay, self.caution, self.cautious_weight_decay, grad, rounding, idx)


class MuonAdamWOracle:
    """heavyball.MuonAdamW (heavyball/__init__.py:475-540) for fp32 gradients: parameters with two or more dimensions go
    through MuonOracle's chain (state ``nesterov_ema_momentum_4``), the others through ``scale_by_adam`` + ``update_param_``,
    which on fp32 is the arithmetic of the fused Adam step (state ``scale_by_adam_exp_avg_0`` / ``_exp_avg_sq_0``).
    Both routes share the group's step counter and learning rate."""

    def __init__(self, params, lr=0.0025, betas=(0.9, 0.99), eps=1e-8, weight_decay=0.0, warmup_steps=0, caution=False,
                 cautious_weight_decay=False, rounding=None, mars=False, mars_gamma=0.0025, ecc=None, storage_dtype="float32",
                 nesterov=True, gradient_clipping=None, update_clipping=None, param_ecc=None):  # fmt: skip
        from .first_order import FirstOrderOracle, narrow_params

        self.params = params
        self.mat_idx = [i for i, p in enumerate(params) if p.dim() >= 2]
        self.vec_idx = [i for i, p in enumerate(params) if p.dim() < 2]
        self.rounding = rounding or HalfRounding()
        params = self.params = narrow_params(params, param_ecc, self.rounding)  # both routes work on the narrowed parameters
        kw = dict(lr=lr, betas=betas, weight_decay=weight_decay, warmup_steps=warmup_steps, caution=caution,
                  cautious_weight_decay=cautious_weight_decay, mars=mars, mars_gamma=mars_gamma, ecc=ecc, storage_dtype=storage_dtype,
                  gradient_clipping=gradient_clipping, update_clipping=update_clipping)  # fmt: skip
        self.muon = MuonOracle(list(params), rounding=self.rounding, nesterov=nesterov, **kw)
        self.muon.KEY = "nesterov_ema_momentum_4" if nesterov else "exp_avg_exp_avg_4"
        self.adam = FirstOrderOracle("adam", list(params), eps=eps, rounding=self.rounding, **kw)
        self.adam.fn_name = "scale_by_adam"
        self.adam.unfused = True  # heavyball/__init__.py:530-533: the route is scale_by_adam -> update_param_, never the fused form
        self.adam.mars_idx = 6  # behind the route's guards (trajectories written from the reference)

    @property
    def state(self):
        return [self.muon.state[i] if i in self.mat_idx else self.adam.state[i] for i in range(len(self.params))]

    def step(self, grads):
        if all(g is None for g in grads):
            return
        from . import first_order as fo

        # both routes side by side: the clips sit around the route (heavyball/chainable.py:2696-2701), so each acts on the
        # tensors of the whole group at once
        fo.run_clip_points([self.muon.step_gen([g if i in self.mat_idx else None for i, g in enumerate(grads)]),
                            self.adam.step_gen([g if i in self.vec_idx else None for i, g in enumerate(grads)])])  # fmt: skip
        # one step counter for the group (heavyball/chainable.py:2531-2570): keep the two halves aligned when one had no gradient
        top = max(int(self.muon.step_count), int(self.adam.step_count))
        self.muon.step_count = torch.tensor(top, dtype=torch.int64)
        self.adam.step_count = torch.tensor(top, dtype=torch.int64)

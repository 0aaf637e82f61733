"""AdamW / LaProp optimizer step, CPU restatement (test infrastructure; see oracle/__init__.py).

Op-for-op restatement, on CPU torch tensors, of the reference's eager path:

  beta_debias                 heavyball/utils.py:337-338
  scalar_guard                heavyball/utils.py:1089-1103   (python floats become fp32 0-d tensors)
  stochastic_lerp / _lerp     heavyball/utils.py:1041-1048, :1842-1849
  exp_avg_sq / eps_sqrt       heavyball/utils.py:413-434
  fused_adam                  heavyball/utils.py:1921-1965
  fused_laprop                heavyball/utils.py:2247-2291
  fused_adopt (+ warm-up)     heavyball/utils.py:2294-2315, heavyball/chainable.py:945-969, :587-610 (WarmupGuard)
  fused_ademamix              heavyball/utils.py:2086-2183, :290-334 (alpha / beta3 schedules)
  fused_nadam                 heavyball/utils.py:341-410, :2003-2083, heavyball/chainable.py:272-274 (mu_product)
  update (weight decay etc.)  heavyball/utils.py:2373-2406
  mars_correction             heavyball/utils.py:3616-3627, called from heavyball/chainable.py:642-647
  cautioning                  heavyball/utils.py:3652-3658
  clipping                    heavyball/utils.py:3226-3297
  step loop                   heavyball/chainable.py:2531-2570 (step counter, lr warm-up), :2292-2323 (chain)

Where the reference takes random numbers, these functions take a ``rounding`` object (oracle/rounding.py).
"""

from typing import List, Optional

import torch
from torch import Tensor

import numpy as np

from . import philox
from .ecc import MODES, EccTensor, copy_stochastic, promote, stochastic_round
from .rounding import HalfRounding


def ieee_sqrt(x: Tensor) -> Tensor:
    """Correctly rounded fp32 square root (float64 hardware sqrt, then one rounding: innocuous for 53 >= 2*24 + 2 bits).

    The one place where this oracle does not call the reference's own ATen op: ``torch.sqrt`` on CPU goes through a
    vendor vector-math library whose result is within 1 ulp but is *not* correctly rounded and differs between CPU
    models (measured: 0.6 % of elements off by one ulp on one host, 17 % on another), so it cannot serve as a
    bit-level anchor.  The correctly rounded value is the one every such implementation approximates; results of
    the reference itself therefore agree with this oracle to ~1 ulp per step, not bit for bit.
    """
    return torch.from_numpy(np.sqrt(x.detach().numpy().astype(np.float64)).astype(np.float32)).view(x.shape)


def f32(x) -> Tensor:
    """scalar_guard for a python float (heavyball/utils.py:1093-1094)."""
    return torch.empty((), dtype=torch.float32).fill_(x)


def beta_debias(beta, step):
    """heavyball/utils.py:337-338, evaluated on whatever it is given (fp32 0-d tensors on the hot path)."""
    return 1 - (1 - beta) / (1 - beta**step)


def step_lr(base_lr: float, step: Tensor, warmup_steps: int) -> Tensor:
    """heavyball/chainable.py:2560: fp32 0-d tensor, since ``step`` is an int64 0-d tensor."""
    return base_lr * step / step.clamp(min=warmup_steps + 1)


def stochastic_lerp_(x: List, y: List[Tensor], a, rounding, stream, tidx):
    """heavyball/utils.py:1041-1048: x <- x*(1-a) + y*a, written through copy_stochastic."""
    for x_, y_, t in zip(x, y, tidx):
        x32 = promote(x_)
        y32 = promote(y_)
        if x32.dtype != y32.dtype:
            y32 = y32.to(x32.dtype)
        copy_stochastic(x_, x32 * (1 - a) + y32 * a, rounding, stream, t)


def lerp_(state: List, grad: List[Tensor], beta, rounding, stream, tidx) -> List[Tensor]:
    """heavyball/utils.py:1842-1849: returns the fp32 state *before* it is re-encoded."""
    ea32 = [promote(s) for s in state]
    grad = [promote(g) for g in grad]
    a = 1 - beta
    # ea32 holds plain fp32 tensors, so the inner copy_stochastic is a plain copy
    stochastic_lerp_(ea32, grad, a, rounding, stream, tidx)
    for s, e, t in zip(state, ea32, tidx):
        if s is not e:
            copy_stochastic(s, e, rounding, stream, t)
    return ea32


def exp_avg_sq_(state: List, grad: List[Tensor], beta2, eps, rounding, tidx) -> List[Tensor]:
    """heavyball/utils.py:417-434 with out=[None]: v <- lerp(v, g*g); returns max(sqrt(v), eps)."""
    g32 = [promote(g) for g in grad]
    s32 = lerp_(state, [g_ * g_ for g_ in g32], beta2, rounding, philox.STREAM_EXP_AVG_SQ, tidx)
    return [ieee_sqrt(d).clamp(min=eps) for d in s32]


def cautioning(g: Tensor, update: Tensor) -> Tensor:
    """heavyball/utils.py:3652-3658."""
    mask = g.signbit() ^ update.signbit()
    update = update.masked_fill(mask, 0)
    scale = mask.numel() / (mask.numel() - mask.sum()).clamp(min=1)
    update.mul_(scale)
    return update


def update_(p: List, u: List[Tensor], decay, lr, caution: bool, cautious_decay: bool, g: List[Optional[Tensor]], rounding, tidx):
    """heavyball/utils.py:2373-2390: p <- p*(1 - d*lr) + u*(-lr), written through copy_stochastic."""
    for u_, g_, p_, t in zip(u, g, p, tidx):
        u_ = promote(u_.view(p_.shape))
        p32_ = promote(p_)
        if caution:
            u_ = cautioning(g_, u_)
        d = decay * (1 - (p32_.signbit() ^ u_.signbit()).to(p32_.dtype)) if cautious_decay else decay
        p32_ = p32_ * (1 - d * lr) + u_ * -lr
        copy_stochastic(p_, p32_, rounding, philox.STREAM_PARAM, t)


def update_param_(param, update, lr, decay, caution=False, cautious_decay=False, grad=None, rounding=None, tidx=None):
    """heavyball/utils.py:2393-2406: the non-fused tail of chain(); ``decay`` stays a python float here."""
    lr = lr.to(torch.float32) if isinstance(lr, Tensor) else f32(lr)
    if not caution:
        grad = [None] * len(param)
    update_(param, update, decay, lr, caution, cautious_decay, grad, rounding or HalfRounding(), tidx or list(range(len(param))))


def fused_adam_(y, exp_avg, exp_avg_sq, update, grad, beta1, beta2, step, lr, eps, decay, caution, cautious_decay, rounding, tidx):
    """heavyball/utils.py:1946-1965 then :1921-1943.  ``eps`` stays a python float (:1961-1962)."""
    beta1, beta2, lr, decay = f32(beta1), f32(beta2), lr.to(torch.float32), f32(decay)
    beta1 = beta_debias(beta1, step)
    beta2 = beta_debias(beta2, step)
    u32 = [promote(u) for u in update]
    g32 = [promote(g) for g in grad]
    exp_avg32 = lerp_(exp_avg, u32, beta1, rounding, philox.STREAM_EXP_AVG, tidx)
    denom = exp_avg_sq_(exp_avg_sq, u32, beta2, eps, rounding, tidx)
    update_(y, [e_ / d_ for e_, d_ in zip(exp_avg32, denom)], decay, lr, caution, cautious_decay, g32, rounding, tidx)


def fused_laprop_(y, exp_avg, exp_avg_sq, update, grad, beta1, beta2, step, lr, decay, caution, cautious_decay, rounding, tidx, eps=1e-8):
    """heavyball/utils.py:2272-2291 then :2247-2269.  v first, then m on the normalised gradient."""
    beta1, beta2, lr, eps, decay = f32(beta1), f32(beta2), lr.to(torch.float32), f32(eps), f32(decay)
    beta1 = beta_debias(beta1, step)
    beta2 = beta_debias(beta2, step)
    u32 = [promote(u) for u in update]
    gp32 = [promote(g) for g in grad]
    denom = exp_avg_sq_(exp_avg_sq, u32, beta2, eps, rounding, tidx)
    u32 = lerp_(exp_avg, [u_ / d_ for u_, d_ in zip(u32, denom)], beta1, rounding, philox.STREAM_EXP_AVG, tidx)
    update_(y, u32, decay, lr, caution, cautious_decay, gp32, rounding, tidx)


def fused_adopt_(y, update, grad, exp_avg_sq, exp_avg, beta1, beta2, step, lr, eps, decay, caution, cautious_decay, rounding, tidx,
                 apply=True):  # fmt: skip
    """heavyball/utils.py:2307-2315 then :2294-2304.  ``step`` is the group's step minus one (heavyball/chainable.py:961);
    ``eps`` stays a python float.  The update uses the second moment of the steps before; that moment is advanced last.
    ``apply=False`` is the un-fused ``adopt`` (:2319-2334): the same moments, the update returned instead of applied."""
    beta1, beta2, lr, decay = f32(beta1), f32(beta2), lr.to(torch.float32), f32(decay)
    u32 = [promote(u) for u in update]
    g32 = [promote(g) for g in grad]
    v32 = [promote(v) for v in exp_avg_sq]
    b1 = beta_debias(beta1, step)
    m_new = lerp_(exp_avg, [u_ / ieee_sqrt(d_).clamp(min=eps) for u_, d_ in zip(u32, v32)], b1, rounding, philox.STREAM_EXP_AVG, tidx)
    if apply:
        update_(y, m_new, decay, lr, caution, cautious_decay, g32, rounding, tidx)
    b2 = beta_debias(beta2, step + 1)
    stochastic_lerp_(exp_avg_sq, [u_ * u_ for u_ in u32], 1 - b2, rounding, philox.STREAM_EXP_AVG_SQ, tidx)
    return m_new


def adopt_warmup_(exp_avg_sq, update, rounding, tidx):
    """heavyball/chainable.py:945-946 -> heavyball/utils.py:436-454 with beta2 = 0 (an int, so an int64 0-d tensor after
    scalar_guard): v <- v*0 + u*u*1.  The scaled update it also produces is dropped (WarmupGuard skips the update)."""
    beta2 = torch.zeros((), dtype=torch.int64)
    lerp_(exp_avg_sq, [promote(u) * promote(u) for u in update], beta2, rounding, philox.STREAM_EXP_AVG_SQ, tidx)


def linear_warmup_scheduler(step: int, alpha_end: float, alpha_start: float = 0.0, warmup=None) -> float:
    """heavyball/utils.py:290-298 (python floats)."""
    if warmup is None or warmup <= 0:
        return alpha_end
    if step < warmup:
        a = step / float(warmup)
        return (1.0 - a) * alpha_start + a * alpha_end
    return alpha_end


def linear_hl_warmup_scheduler(step: int, beta_end: float, beta_start: float, warmup=None, eps: float = 1e-8) -> float:
    """heavyball/utils.py:301-318: interpolates the half-life, not beta (python floats)."""
    import math

    if warmup is None or warmup <= 0:
        return beta_end
    if step < warmup:
        a = step / float(warmup)
        hl0 = math.log(0.5) / math.log(beta_start + eps) - 1
        hl1 = math.log(0.5) / math.log(beta_end + eps) - 1
        beta = math.pow(0.5, 1.0 / ((1.0 - a) * hl0 + a * hl1 + 1.0))
        return min(max(beta, 0.0), 1.0 - eps)
    return beta_end


def fused_ademamix_(y, exp_avg_fast, exp_avg_slow, exp_avg_sq, update, grad, betas, step, lr, eps, decay, alpha, caution,
                    cautious_decay, beta3_warmup, alpha_warmup, rounding, tidx, apply=True):  # fmt: skip
    """heavyball/utils.py:2135-2183 then :2086-2132.  Every scalar goes through scalar_guard here (eps too).
    ``apply=False`` is the un-fused ``ademamix_`` (:2186-2210): the update is returned instead of applied."""
    beta1, beta2, beta3_final = betas
    alpha_f = linear_warmup_scheduler(int(step), alpha_end=alpha, alpha_start=0.0, warmup=alpha_warmup)
    beta3_f = linear_hl_warmup_scheduler(int(step), beta_end=beta3_final, beta_start=beta1, warmup=beta3_warmup)
    beta1, beta2, beta3, alpha_t, lr, eps, decay = f32(beta1), f32(beta2), f32(beta3_f), f32(alpha_f), lr.to(torch.float32), f32(eps), f32(decay)
    b1 = beta_debias(beta1, step)
    b2 = beta_debias(beta2, step)
    u32 = [promote(u) for u in update]
    g32 = [promote(g) for g in grad]
    fast32 = lerp_(exp_avg_fast, u32, b1, rounding, philox.STREAM_EXP_AVG, tidx)
    slow32 = lerp_(exp_avg_slow, u32, beta3, rounding, philox.STREAM_EXP_AVG_SLOW, tidx)
    denom = exp_avg_sq_(exp_avg_sq, u32, b2, eps, rounding, tidx)
    out = [(f_ + s_ * alpha_t) / d_ for f_, s_, d_ in zip(fast32, slow32, denom)]
    if apply:
        update_(y, out, decay, lr, caution, cautious_decay, g32, rounding, tidx)
    return out


def nadam_moments(beta1: Tensor, step: Tensor, momentum_decay: float):
    """heavyball/utils.py:341-347."""
    md = torch.as_tensor(momentum_decay, dtype=beta1.dtype)
    base = torch.tensor(0.96, dtype=beta1.dtype)
    step_f = step.to(beta1.dtype)
    mu = beta1 * (1 - 0.5 * torch.pow(base, step_f * md))
    mu_next = beta1 * (1 - 0.5 * torch.pow(base, (step_f + 1) * md))
    return mu, mu_next


def fma_(u: Tensor, p: Tensor, alpha: float) -> Tensor:
    """``u.add_(p, alpha=alpha)`` as one fused multiply-add per element: what ATen computes on a GPU and in the vector body of
    its CPU loop (``vec::fmadd``; only the scalar tail of the CPU loop rounds the product first).  float64 holds the
    product of two fp32 numbers exactly; the sum then rounds twice (53 bits, then 24), which differs from a single
    rounding only when the 53-bit sum lands exactly on an fp32 tie - never seen on the test sizes."""
    a = np.float64(np.float32(alpha))
    return torch.from_numpy((p.numpy().astype(np.float64) * a + u.numpy().astype(np.float64)).astype(np.float32)).view(u.shape)


def fused_nadam_(param, exp_avg, exp_avg_sq, mu_product, update, grad, beta1, beta2, step, lr, eps, momentum_decay, weight_decay,
                 decoupled_weight_decay, caution, cautious_decay, rounding, tidx, apply=True):  # fmt: skip
    """heavyball/utils.py:2046-2083 then :2003-2043 with the helpers of :350-410.  Without ``decoupled_weight_decay`` the
    decay enters as ``weight_decay * p`` added to the gradient (and to the gradient caution compares with) and is taken
    out of the finished update again; the parameter update itself then runs with decay 0.
    ``apply=False`` is the un-fused ``nadam_`` (:1968-2000): the gradient that caution compares with is left alone
    (``_nadam_prepare_weight_decay`` gets no gradient) and the update is returned instead of applied."""
    beta1_t, beta2_t, lr, eps_t = f32(beta1), f32(beta2), lr.to(torch.float32), f32(eps)
    mu, mu_next = nadam_moments(beta1_t, step, momentum_decay)
    wd = float(weight_decay)
    u32 = [promote(u) for u in update]
    g32 = [promote(g) for g in grad]
    p32 = [promote(p) for p in param]
    coupled = wd != 0 and not decoupled_weight_decay
    decay = wd if (wd != 0 and decoupled_weight_decay) else 0.0
    if coupled:
        u32 = [fma_(u_, p_, wd) for u_, p_ in zip(u32, p32)]
        g32 = [fma_(g_, p_, wd) for g_, p_ in zip(g32, p32)]
    exp_avg32 = lerp_(exp_avg, u32, beta1_t, rounding, philox.STREAM_EXP_AVG, tidx)  # beta1 is not debiased here (:394)
    denom = exp_avg_sq_(exp_avg_sq, u32, beta_debias(beta2_t, step), eps_t, rounding, tidx)
    for mp_ in mu_product:
        mp_.mul_(mu)
    one = torch.ones((), dtype=torch.float32)
    grad_scale = one - mu
    out = []
    for u_, e_, d_, mp_ in zip(u32, exp_avg32, denom, mu_product):
        mp32 = promote(mp_)
        gw = grad_scale / (one - mp32)
        ew = mu_next / (one - mp32 * mu_next)
        out.append(u_ / d_ * gw + e_ / d_ * ew)
    if coupled:
        out = [o_ - p_ * wd for o_, p_ in zip(out, p32)]
    if apply:
        update_(param, out, f32(decay), lr, caution, cautious_decay, g32, rounding, tidx)
    return out


def mars_correction(g: List[Tensor], old_g: List, beta1, gamma, rounding, tidx):
    """heavyball/utils.py:3623-3627 and :3616-3620.

    The argument names are the reference's; heavyball/chainable.py:645 passes (mars_gamma, beta1) into
    (beta1, gamma), which this oracle's caller reproduces.
    """
    a = f32(-gamma * beta1 / (1 - beta1))
    g_copy = [g_.clone() for g_ in g]
    stochastic_lerp_(g, old_g, a, rounding, philox.STREAM_MARS_SR, tidx)
    for o, c, t in zip(old_g, g_copy, tidx):
        copy_stochastic(o, c, rounding, philox.STREAM_OLD_GRAD, t)


# ---------------------------------------------------------------------------------------------------------
# clipping (heavyball/utils.py:3226-3297)
# ---------------------------------------------------------------------------------------------------------
def _clip(x: Tensor, norm: Tensor, clip_at, eps=1e-8) -> Tensor:
    """heavyball/utils.py:3226-3232; returns the clipped fp32 tensor."""
    x32 = promote(x)
    norm = clip_at / norm.clamp(min=max(clip_at, eps))
    return x32 * norm


def l2_clip(xs: List[Tensor], clip_at=1.0, eps=1e-8) -> List[Tensor]:
    """heavyball/utils.py:3235-3250."""
    return [_clip(x, promote(x).norm(), clip_at, eps) for x in xs]


def rmsnorm_clip(xs: List[Tensor], clip_at=1.0, eps=1e-8) -> List[Tensor]:
    """heavyball/utils.py:3253-3262."""
    return [_clip(x, promote(x).square().mean().sqrt(), clip_at, eps) for x in xs]


def global_l2norm_clip(xs: List[Tensor], clip_at=1.0, eps=1e-8) -> List[Tensor]:
    """heavyball/utils.py:3283-3297."""
    clip_at = f32(clip_at)
    norm = 0
    for i in xs:
        norm += promote(i).square().sum()
    norm = norm**0.5
    scalar = clip_at / norm.clamp(min=max(clip_at, eps))
    return [promote(x) * scalar for x in xs]


def global_rmsnorm_clip(xs: List[Tensor], clip_at=1.0, eps=1e-8) -> List[Tensor]:
    """heavyball/utils.py:3265-3280."""
    clip_at = f32(clip_at)
    norm = 0
    numel = sum(i.numel() for i in xs)
    for i in xs:
        norm += promote(i).square().sum()
    norm = (norm / numel) ** 0.5
    scalar = clip_at / norm.clamp(min=max(clip_at, eps))
    return [promote(x) * scalar for x in xs]


def run_clip_points(gens):
    """Runs step generators side by side.  Each yields ``(clip kind, tensors, tensor indices)`` where the reference's chain clips
    (heavyball/chainable.py:2696-2701) and is sent its tensors back clipped.  The generators of one parameter group (the two routes
    of MuonAdamW) reach their clip points in the same order, and each point is clipped once over the tensors of all of them, in the
    order of the group's parameters: the reference's chain places the clips around the route."""
    fns = {"l2_clip_": l2_clip, "rmsnorm_clip_": rmsnorm_clip, "global_l2norm_clip": global_l2norm_clip, "global_rmsnorm_clip": global_rmsnorm_clip}
    waiting = []
    for g in gens:
        try:
            waiting.append((g, next(g)))
        except StopIteration:
            pass
    while waiting:
        kind = waiting[0][1][0]
        assert all(r[0] == kind for _, r in waiting)
        merged = sorted(((t, k, j) for k, (_, r) in enumerate(waiting) for j, t in enumerate(r[2])))
        out = fns[kind]([waiting[k][1][1][j] for _, k, j in merged])
        back = [[None] * len(r[1]) for _, r in waiting]
        for (_, k, j), c in zip(merged, out):
            back[k][j] = c
        nxt = []
        for (g, _), b in zip(waiting, back):
            try:
                nxt.append((g, g.send(b)))
            except StopIteration:
                pass
        waiting = nxt


# ---------------------------------------------------------------------------------------------------------
# The step loop of one param group
# ---------------------------------------------------------------------------------------------------------
def palm_betas(betas, step: Tensor, beta2_scale: float):
    """heavyball/chainable.py:1921-1925 (``palm_beta2``, first in the chain: :2693-2694): beta2 = 1 - step ** -beta2_scale
    on the int64 step tensor, i.e. an fp32 0-d tensor, written back into the group's betas."""
    beta2 = 1 - step ** -beta2_scale
    return (betas[0], beta2, *betas[2:])


def narrow_params(params, param_ecc, rounding):
    """heavyball/chainable.py:2421-2444: param_ecc narrows the live parameter at construction (a parameter that already is an
    EccTensor, or param_ecc None: unchanged)."""
    out = []
    for i, p in enumerate(params):
        if param_ecc is None or isinstance(p, EccTensor):
            out.append(p)
            continue
        pd, cd = MODES[param_ecc]
        e = EccTensor(p.to(pd), torch.zeros(p.shape, dtype=cd))
        if p.dtype != pd:
            e.compute_correction(p.float(), rounding.at_step(0).uniform(philox.STREAM_INIT_PARAM, i, p.shape))
        out.append(e)
    return out


class FirstOrderOracle:
    """AdamW or LaProp over a list of tensors, with the reference's state layout.

    ``state[i]`` is the per-tensor dict the reference keeps under ``opt.state[p][0]`` with the same key
    names (heavyball/chainable.py:73-74, :2368-2382): ``update_by_adam_exp_avg_0`` ... and, with ECC, the
    ``"::ecc"`` siblings; parameters under param_ecc live in ``self.params[i]`` as EccTensor with the correction
    also visible as ``state[i]["param::ecc"]``.
    """

    def __init__(
        self,
        kind: str,
        params: List[Tensor],
        lr=None,
        betas=None,
        eps=1e-8,
        weight_decay=0.0,
        cautious_weight_decay=False,
        warmup_steps=0,
        storage_dtype="float32",
        mars=False,
        caution=False,
        mars_gamma=0.0025,
        ecc=None,
        param_ecc=None,
        rounding=None,
        gradient_clipping=None,
        update_clipping=None,
        alpha=2.0,
        beta3_warmup=None,
        alpha_warmup=None,
        momentum_decay=4e-3,
        decoupled_weight_decay=False,
        palm=False,
        beta2_scale=0.8,
    ):
        assert kind in ("adam", "laprop", "adopt", "ademamix", "nadam")
        clips = (None, "l2_clip_", "rmsnorm_clip_", "global_l2norm_clip", "global_rmsnorm_clip")
        assert gradient_clipping in clips and update_clipping in clips
        self.gradient_clipping, self.update_clipping = gradient_clipping, update_clipping
        self.kind = kind
        self.fn_name = "update_by_" + kind
        # the index the reference's walk gives MARS' guard: behind the guards of the update transform (chainable.py:2347-2382)
        self.mars_idx = {"adam": 2, "laprop": 2, "ademamix": 2, "adopt": 3, "nadam": 3}[kind]
        self.alpha, self.beta3_warmup, self.alpha_warmup = alpha, beta3_warmup, alpha_warmup
        self.momentum_decay, self.decoupled_weight_decay = momentum_decay, decoupled_weight_decay
        self.palm, self.beta2_scale = palm, beta2_scale
        if update_clipping is not None:  # heavyball/chainable.py:2676-2684: the fused transform is swapped for the un-fused one
            self.fn_name = "scale_by_" + kind
        # constructor defaults of heavyball/__init__.py:44-80 (AdamW), :740-776 (LaProp), :640-681 (ADOPT), :124-164, :83-121
        d_lr, d_betas = {"adam": (0.0025, (0.9, 0.99)), "laprop": (0.0025, (0.9, 0.99)), "adopt": (0.0025, (0.9, 0.99)),
                         "ademamix": (0.001, (0.9, 0.999, 0.9999)), "nadam": (0.002, (0.9, 0.999))}[kind]  # fmt: skip
        lr = d_lr if lr is None else lr
        betas = d_betas if betas is None else betas
        self.lr, self.betas, self.eps, self.weight_decay = lr, betas, eps, weight_decay
        self.cautious_weight_decay, self.warmup_steps = cautious_weight_decay, warmup_steps
        self.storage_dtype = getattr(torch, storage_dtype)
        self.mars, self.caution, self.mars_gamma = mars, caution, mars_gamma
        self.ecc, self.param_ecc = ecc, param_ecc
        self.unfused = False  # True: the scale_by_* form of the transform even without update_clipping (MuonAdamW's vector route)
        self.rounding = rounding or HalfRounding()
        self.step_count = torch.zeros((), dtype=torch.int64)
        self.state = [dict() for _ in params]
        self.params = narrow_params(params, param_ecc, self.rounding)
        for i, e in enumerate(self.params):
            if isinstance(e, EccTensor):
                self.state[i]["param::ecc"] = e.corr

    def key(self, name):
        idx = {"mars_old_grad": self.mars_idx, "mu_product": 1}.get(name, 0)
        fn = "mars" if name == "mars_old_grad" else self.fn_name
        return f"{fn}_{name}_{idx}"

    def _state_tensor(self, i, name, ref_shape):
        """ZeroGuard (heavyball/chainable.py:277-301): lazily created zeros, ECC pair when ``ecc`` is set."""
        st = self.state[i]
        k = self.key(name)
        if k not in st:
            if self.ecc is None:
                st[k] = torch.zeros(ref_shape, dtype=self.storage_dtype)
            else:
                e = EccTensor.zeros(ref_shape, self.ecc)
                st[k], st[k + "::ecc"] = e.primary, e.corr
        if self.ecc is None:
            return st[k]
        return EccTensor(st[k], st[k + "::ecc"])

    def step(self, grads: List[Optional[Tensor]]):
        run_clip_points([self.step_gen(grads)])

    def step_gen(self, grads: List[Optional[Tensor]]):
        """The step as a generator: it yields ``(clip kind, tensors)`` at the chain's clip points and is sent the clipped tensors."""
        idx = [i for i, g in enumerate(grads) if g is not None]
        if not idx:
            return
        self.step_count = self.step_count + 1
        step = self.step_count
        self.state[idx[0]]["step"] = step
        lr = step_lr(self.lr, step, self.warmup_steps)
        rounding = self.rounding.at_step(int(step))
        if self.palm:
            self.betas = palm_betas(self.betas, step, self.beta2_scale)
        p = [self.params[i] for i in idx]
        grad = [grads[i] for i in idx]
        update = [g.clone() for g in grad]  # heavyball/chainable.py:2293
        if self.mars:
            old = [self._state_tensor(i, "mars_old_grad", grads[i].shape) for i in idx]
            mars_correction(update, old, self.mars_gamma, self.betas[0], rounding, idx)
            for g_, u_ in zip(grad, update):  # heavyball/chainable.py:646: same dtype, plain copy
                g_.copy_(u_)
        if self.gradient_clipping is not None:
            # heavyball/chainable.py:2696-2699: the clip acts on the update after MARS and before the Adam/LaProp transform;
            # heavyball/utils.py:3226-3232 writes x32 * scale back with copy_stochastic_ (a stochastic round for bf16)
            clipped = yield (self.gradient_clipping, update, idx)
            for j, (u, c) in enumerate(zip(update, clipped)):
                if u.dtype == torch.bfloat16:
                    u.copy_(stochastic_round(c, rounding.noise16(philox.STREAM_CLIP, idx[j], u.shape)))
                else:
                    u.copy_(c.to(u.dtype))
        m = [self._state_tensor(i, "exp_avg", grads[i].shape) for i in idx] if self.kind != "ademamix" else None
        v = [self._state_tensor(i, "exp_avg_sq", grads[i].shape) for i in idx]
        if self.update_clipping is not None or self.unfused:
            # un-fused chain (heavyball/chainable.py:2676-2701): scale_by_* leaves its result in the update buffer, which has the
            # gradient's dtype (copy_stochastic_list_: a stochastic round for bf16, heavyball/utils.py:1868, :2229, :2000, :2209,
            # :2327), the clip rewrites that buffer the same way (:3226-3232), update_param_ applies it (:2393-2406)
            u32 = [promote(u) for u in update]
            if self.kind == "adam":
                b1 = beta_debias(f32(self.betas[0]), step)
                b2 = beta_debias(f32(self.betas[1]), step)
                ea32 = lerp_(m, u32, b1, rounding, philox.STREAM_EXP_AVG, idx)
                denom = exp_avg_sq_(v, u32, b2, f32(self.eps), rounding, idx)
                new = [e_ / d_ for e_, d_ in zip(ea32, denom)]
            elif self.kind == "laprop":
                b1 = beta_debias(f32(self.betas[0]), step)
                b2 = beta_debias(f32(self.betas[1]), step)
                denom = exp_avg_sq_(v, u32, b2, f32(1e-8), rounding, idx)
                new = lerp_(m, [u_ / d_ for u_, d_ in zip(u32, denom)], b1, rounding, philox.STREAM_EXP_AVG, idx)
            elif self.kind == "adopt":
                if min(self.state[i].get("_warmup_1", 0) for i in idx) < 1:  # WarmupGuard, as in the fused chain below
                    adopt_warmup_(v, update, rounding, idx)
                    for i in idx:
                        self.state[i]["_warmup_1"] = self.state[i].get("_warmup_1", 0) + 1
                    return
                # heavyball/chainable.py:1014-1023 passes no eps: the default 1e-8 of heavyball/utils.py:2330
                new = fused_adopt_(None, update, grad, v, m, self.betas[0], self.betas[1], step - 1, lr, 1e-8, 0.0, False, False,
                                   rounding, idx, apply=False)  # fmt: skip
            elif self.kind == "ademamix":
                fast = [self._state_tensor(i, "exp_avg_fast", grads[i].shape) for i in idx]
                slow = [self._state_tensor(i, "exp_avg_slow", grads[i].shape) for i in idx]
                new = fused_ademamix_(None, fast, slow, v, update, grad, self.betas, step, lr, self.eps, 0.0, self.alpha, False, False,
                                      self.beta3_warmup, self.alpha_warmup, rounding, idx, apply=False)  # fmt: skip
            else:
                k = self.key("mu_product")
                for i in idx:
                    if k not in self.state[i]:
                        self.state[i][k] = torch.ones((), dtype=self.storage_dtype)
                new = fused_nadam_(p, m, v, [self.state[i][k] for i in idx], update, grad, self.betas[0], self.betas[1], step, lr, self.eps,
                                   self.momentum_decay, self.weight_decay, self.decoupled_weight_decay, False, False, rounding, idx,
                                   apply=False)  # fmt: skip
            for u, n, t in zip(update, new, idx):
                copy_stochastic(u, n, rounding, philox.STREAM_UPDATE, t)
            if self.update_clipping is not None:
                clipped = yield (self.update_clipping, update, idx)
                for u, c, t in zip(update, clipped, idx):
                    copy_stochastic(u, c, rounding, philox.STREAM_UPDATE_CLIP, t)
            # the tail of the chain decays with the group's weight_decay whatever the transform did with it (NAdam: on top of its own)
            update_param_(p, update, lr, self.weight_decay, self.caution, self.cautious_weight_decay, grad, rounding, idx)
            return
        if self.kind == "adopt":
            # WarmupGuard (heavyball/chainable.py:597-610): while any tensor of this call has not had its warm-up, every
            # tensor of the call takes the warm-up function and the update is skipped
            if min(self.state[i].get("_warmup_1", 0) for i in idx) < 1:
                adopt_warmup_(v, update, rounding, idx)
                for i in idx:
                    self.state[i]["_warmup_1"] = self.state[i].get("_warmup_1", 0) + 1
                return
            fused_adopt_(p, update, grad, v, m, self.betas[0], self.betas[1], step - 1, lr, self.eps, self.weight_decay,
                         self.caution, self.cautious_weight_decay, rounding, idx)  # fmt: skip
        elif self.kind == "ademamix":
            fast = [self._state_tensor(i, "exp_avg_fast", grads[i].shape) for i in idx]
            slow = [self._state_tensor(i, "exp_avg_slow", grads[i].shape) for i in idx]
            fused_ademamix_(p, fast, slow, v, update, grad, self.betas, step, lr, self.eps, self.weight_decay, self.alpha,
                            self.caution, self.cautious_weight_decay, self.beta3_warmup, self.alpha_warmup, rounding, idx)  # fmt: skip
        elif self.kind == "nadam":
            k = self.key("mu_product")
            for i in idx:  # heavyball/chainable.py:272-274: a 0-d tensor of ones in the storage dtype, never an ECC pair
                if k not in self.state[i]:
                    self.state[i][k] = torch.ones((), dtype=self.storage_dtype)
            fused_nadam_(p, m, v, [self.state[i][k] for i in idx], update, grad, self.betas[0], self.betas[1], step, lr, self.eps,
                         self.momentum_decay, self.weight_decay, self.decoupled_weight_decay, self.caution,
                         self.cautious_weight_decay, rounding, idx)  # fmt: skip
        elif self.kind == "adam":
            fused_adam_(p, m, v, update, grad, self.betas[0], self.betas[1], step, lr, self.eps, self.weight_decay,
                        self.caution, self.cautious_weight_decay, rounding, idx)  # fmt: skip
        else:
            fused_laprop_(p, m, v, update, grad, self.betas[0], self.betas[1], step, lr, self.weight_decay,
                          self.caution, self.cautious_weight_decay, rounding, idx)  # fmt: skip

    def param_f32(self, i) -> Tensor:
        return promote(self.params[i])

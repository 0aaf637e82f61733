"""Writes the golden fixtures in this directory from the reference implementation.

Run ONCE in the build container, where the reference tree is mounted at /root/reference:

    python tests/golden/make_golden.py

The reference is imported on CPU with compilation switched off, exactly as its own CPU tests do
(test/test_utils_cpu.py:41-46).  Only inputs and outputs are stored (small tensors, key strings and fp32 bit
patterns); no reference source travels.  The fixtures pin what reading the source cannot:

  layout.json      state_dict key strings, param_group keys and the "heavyball" sub-dict for each optimizer
  scalars.json     bit patterns of the fp32 step scalars (debiased betas, lr with warm-up) for steps 1..30
  ecc.pt           ECC encode/decode vectors for all four modes, with a recorded uniform tensor
  traj_*.pt        three-to-five-step trajectories of AdamW / LaProp variants on tiny tensors, with the reference's
                   random draws replaced by constants (uniform 0.5, 16-bit noise 0x8000) or by recorded tensors
  ns5.pt, muon_*.pt, soap_*.pt   see the functions below

Stochastic sites are made deterministic by replacing ``torch.rand_like`` / ``torch.randint_like`` while
the reference runs; the replacement is visible in this file.
"""

import contextlib
import json
import os
import sys

os.environ["TORCH_COMPILE_DISABLE"] = "1"
HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, "/root/reference")

import torch  # noqa: E402

import heavyball  # noqa: E402
import heavyball.utils  # noqa: E402
from heavyball import chainable as C  # noqa: E402

heavyball.utils.compile_mode = None
torch.set_num_threads(1)


@contextlib.contextmanager
def half_rounding():
    """uniform -> 0.5, 16-bit noise -> 0x8000 for every stochastic site of the reference."""
    rl, ril = torch.rand_like, torch.randint_like
    torch.rand_like = lambda x, *a, **k: torch.full_like(x, 0.5)
    torch.randint_like = lambda x, *a, **k: torch.full_like(x, 1 << 15)
    try:
        yield
    finally:
        torch.rand_like, torch.randint_like = rl, ril


def hexf(t):
    return "%08x" % (t.detach().to(torch.float32).view(torch.int32).item() & 0xFFFFFFFF)


def flat_state(opt, p):
    """The state of a parameter under its plain keys; the states of the further blocks of a split parameter
    (heavyball/utils.py:1612-1623: one state per view) under ``block<k>/<key>``."""
    out = {}
    for idx, st in opt.state[p].items():
        if isinstance(st, dict):
            for k, v in st.items():
                out[k if idx == 0 else f"block{idx}/{k}"] = v
    return out


# ------------------------------------------------------------------------------------------------------
def make_layout():
    out = {}

    def record(name, opt, params):
        for p in params:
            p.grad = torch.randn_like(p.float()).to(p.dtype) * 1e-2
        with half_rounding():
            opt.step()
            for p in params:
                p.grad = torch.randn_like(p.float()).to(p.dtype) * 1e-2
            opt.step()
        sd = opt.state_dict()
        entry = {
            "state_keys": {},
            "param_group_keys": sorted(sd["param_groups"][0].keys()),
            "param_group_values": {
                k: (v if isinstance(v, (int, float, str, bool, type(None))) else repr(v))
                for k, v in sd["param_groups"][0].items()
                if k != "params"
            },
            "heavyball_keys": sorted(sd["heavyball"].keys()),
            "grad_is_none_after_step": all(p.grad is None for p in params),
            "param_dtypes": [str(p.dtype) for p in params],
        }
        for pi, st in sd["state"].items():
            e = {}
            for view, d in st.items():
                def spec(v):
                    if isinstance(v, torch.Tensor):
                        return {"dtype": str(v.dtype), "shape": list(v.shape)}
                    if isinstance(v, (list, tuple)):
                        return [spec(x) for x in v]
                    return repr(sorted(v) if isinstance(v, set) else v)

                e[str(view)] = {k: spec(v) for k, v in d.items()}
            entry["state_keys"][str(pi)] = e
        out[name] = entry

    def ps():
        torch.manual_seed(0)
        return [torch.nn.Parameter(torch.randn(8, 16)), torch.nn.Parameter(torch.randn(16))]

    p = ps(); record("AdamW", heavyball.AdamW(p), p)  # noqa: E702
    p = ps(); record("AdamW_mars", heavyball.AdamW(p, mars=True), p)  # noqa: E702
    p = ps(); record("AdamW_ecc", heavyball.AdamW(p, ecc="bf16+8"), p)  # noqa: E702
    p = ps(); record("AdamW_mars_caution_ecc_paramecc", heavyball.AdamW(p, mars=True, caution=True, ecc="bf16+8", param_ecc="bf16+8"), p)  # noqa: E702,E501
    p = ps(); record("LaProp", heavyball.LaProp(p), p)  # noqa: E702
    p = ps(); record("LaProp_ecc", heavyball.LaProp(p, ecc="bf16+8"), p)  # noqa: E702
    p = ps(); record("LaProp_bf16_storage", heavyball.LaProp(p, storage_dtype="bfloat16"), p)  # noqa: E702
    p = ps(); record("Muon", heavyball.Muon(p), p)  # noqa: E702
    p = ps(); record("SOAP", heavyball.SOAP(p), p)  # noqa: E702
    p = ps(); record("MuonAdamW", heavyball.MuonAdamW(p), p)  # noqa: E702
    p = ps(); record("ADOPT", heavyball.ADOPT(p), p)  # noqa: E702
    p = ps(); record("ADOPT_mars_ecc", heavyball.ADOPT(p, mars=True, ecc="bf16+8"), p)  # noqa: E702
    p = ps(); record("AdEMAMix", heavyball.AdEMAMix(p), p)  # noqa: E702
    p = ps(); record("AdEMAMix_ecc", heavyball.AdEMAMix(p, ecc="bf16+8"), p)  # noqa: E702
    p = ps(); record("NAdam", heavyball.NAdam(p), p)  # noqa: E702
    p = ps(); record("NAdam_ecc", heavyball.NAdam(p, ecc="bf16+8"), p)  # noqa: E702
    with open(os.path.join(HERE, "layout.json"), "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)


# ------------------------------------------------------------------------------------------------------
def make_scalars():
    """fp32 bit patterns of the per-step scalars, computed by the reference's own functions on 0-d tensors."""
    out = {}
    ref = torch.zeros(1)
    for b1, b2 in [(0.9, 0.999), (0.9, 0.99), (0.95, 0.95), (0.9, 0.95)]:
        rows = []
        for s in range(1, 31):
            beta1, beta2, step = heavyball.utils.scalar_guard(b1, b2, s, ref)
            d1 = heavyball.utils.beta_debias(beta1, step)
            d2 = heavyball.utils.beta_debias(beta2, step)
            rows.append([hexf(d1), hexf(1 - d1), hexf(1 - (1 - d1)), hexf(d2), hexf(1 - d2), hexf(1 - (1 - d2))])
        out[f"betas_{b1}_{b2}"] = rows
    for base_lr, warm in [(1e-3, 0), (0.0025, 0), (0.0025, 3), (3e-3, 10)]:
        rows = []
        for s in range(1, 31):
            step = torch.tensor(s, dtype=torch.int64)
            lr = base_lr * step / step.clamp(min=warm + 1)
            rows.append(hexf(lr))
        out[f"lr_{base_lr}_{warm}"] = rows
    # MARS coefficient as the reference computes it (argument order of chainable.py:645)
    g = [torch.zeros(1)]
    a = -0.9 * 0.0025 / (1 - 0.0025)
    out["mars_a_default"] = hexf(heavyball.utils.scalar_guard(a, g[0]))
    with open(os.path.join(HERE, "scalars.json"), "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)


# ------------------------------------------------------------------------------------------------------
def make_ecc():
    out = {}
    gen = torch.Generator().manual_seed(1234)
    specials = torch.tensor(
        [0.0, -0.0, 1.0, -1.0, 1e4, -1e4, 3e10, -3e10, 1e-10, -1e-10, 1e-38, -1e-38, 1e-40, 3e-45, 65504.0, 1e-7, 6e-8, 255.99, 0.1, 1.0 / 3.0],
        dtype=torch.float32,
    )  # fmt: skip
    x = torch.cat([torch.randn(236, generator=gen) * torch.exp(torch.randn(236, generator=gen) * 6), specials])
    u = torch.rand(x.shape, generator=gen)
    out["x"], out["u"] = x, u
    for mode, (pd, cd) in C.ECCConfig._MODES.items():
        cfg = C.ECCConfig(mode)
        xn = x.to(pd)
        corr = torch.zeros(x.shape, dtype=cd)
        st = heavyball.utils._ULPState(corr, cfg.smax)
        rl = torch.rand_like
        torch.rand_like = lambda s, *a, **k: u.clone()
        try:
            st.encode(x, xn)
        finally:
            torch.rand_like = rl
        out[f"{mode}/primary"] = xn.clone()
        out[f"{mode}/corr"] = corr.clone()
        out[f"{mode}/decoded"] = st.decode(xn).clone()
        out[f"{mode}/log_ulp"] = heavyball.utils._log_ulp(xn).clone()
    # bf16 stochastic rounding with recorded noise
    noise = torch.randint(0, 1 << 16, x.shape, generator=gen, dtype=torch.int32)
    ril = torch.randint_like
    torch.randint_like = lambda s, *a, **k: noise.clone()
    try:
        out["sr/noise"] = noise
        out["sr/out"] = heavyball.utils.stochastic_round_(x.clone())
    finally:
        torch.randint_like = ril
    torch.save(out, os.path.join(HERE, "ecc.pt"))


# ------------------------------------------------------------------------------------------------------
def run_traj(name, cls, kwargs, shapes, grad_dtype, steps, grad_scale=1e-2, param_scale=0.02, none_grad_for=None, mode=None, param_dtype=None):
    if mode is not None:  # heavyball.utils.zeroth_power_mode for the length of the run, recorded as meta/zeroth_power_mode
        before, heavyball.utils.zeroth_power_mode = heavyball.utils.zeroth_power_mode, mode
        try:
            run_traj(name, cls, kwargs, shapes, grad_dtype, steps, grad_scale, param_scale, none_grad_for)
        finally:
            heavyball.utils.zeroth_power_mode = before
        path = os.path.join(HERE, f"traj_{name}.pt")
        out = torch.load(path, weights_only=True)
        out["meta/zeroth_power_mode"] = mode
        torch.save(out, path)
        return
    gen = torch.Generator().manual_seed(0)
    params = [torch.nn.Parameter((torch.randn(s, generator=gen) * param_scale).to(param_dtype or torch.float32)) for s in shapes]
    for p in params:
        p.grad_dtype = None  # torch >= 2.9 refuses a gradient of another dtype otherwise
    out = {"meta/name": name, "meta/kwargs": json.dumps(kwargs), "meta/cls": cls.__name__, "meta/steps": steps}
    for i, p in enumerate(params):
        out[f"init/p{i}"] = p.detach().clone()
    with half_rounding():
        opt = cls(params, **kwargs)
        for k in range(1, steps + 1):
            g = torch.Generator().manual_seed(1000 + k)
            for i, p in enumerate(params):
                gr = (torch.randn(p.shape, generator=g) * grad_scale).to(grad_dtype)
                out[f"step{k}/g{i}"] = gr.clone()
                if none_grad_for is not None and i == none_grad_for and k == 1:
                    p.grad = None
                else:
                    p.grad = gr.clone()
            opt.step()
            for i, p in enumerate(params):
                out[f"step{k}/p{i}"] = p.detach().clone()
                for kk, v in flat_state(opt, p).items():
                    if isinstance(v, torch.Tensor):
                        out[f"step{k}/state{i}/{kk}"] = v.detach().clone()
                    elif isinstance(v, (list, tuple)):
                        for li, lv in enumerate(v):
                            if isinstance(lv, torch.Tensor):
                                out[f"step{k}/state{i}/{kk}/{li}"] = lv.detach().clone()
        for i, p in enumerate(params):  # which transforms count as initialised (heavyball/chainable.py:117-133)
            inited = flat_state(opt, p).get("is_initialized")
            if inited is not None:
                out[f"final/is_initialized{i}"] = torch.tensor(sorted(inited), dtype=torch.int64)
    torch.save(out, os.path.join(HERE, f"traj_{name}.pt"))


def make_trajectories():
    shapes = [(4, 8), (16,), (3, 5)]
    A, L = heavyball.AdamW, heavyball.LaProp
    run_traj("adamw_fp32", A, dict(lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01), shapes, torch.float32, 5)
    run_traj("adamw_default", A, dict(), shapes, torch.float32, 3)
    run_traj("laprop_ecc", L, dict(ecc="bf16+8"), shapes, torch.bfloat16, 5, grad_scale=1e-3)
    run_traj("laprop_fp32", L, dict(weight_decay=0.1), shapes, torch.float32, 3)
    run_traj("adamw_mars_caution_ecc_paramecc", A, dict(mars=True, caution=True, ecc="bf16+8", param_ecc="bf16+8"),
             shapes, torch.bfloat16, 5, grad_scale=1e-3)  # fmt: skip
    run_traj("adamw_mars_fp32", A, dict(mars=True, weight_decay=0.01), shapes, torch.float32, 3)
    run_traj("adamw_caution_cwd_warmup", A, dict(caution=True, weight_decay=0.1, cautious_weight_decay=True, warmup_steps=3),
             shapes, torch.float32, 5)  # fmt: skip
    run_traj("laprop_bf16_storage", L, dict(storage_dtype="bfloat16"), shapes, torch.float32, 3)
    run_traj("laprop_ecc_fp16_16", L, dict(ecc="fp16+16", weight_decay=0.01), shapes, torch.float32, 3)
    run_traj("adamw_ecc_bf16_16_paramecc_fp16_8", A, dict(ecc="bf16+16", param_ecc="fp16+8", mars=True), shapes, torch.float32, 3)
    run_traj("adamw_mars_ecc_fp32grad", A, dict(mars=True, ecc="bf16+8"), shapes, torch.float32, 3)
    run_traj("laprop_none_grad", L, dict(ecc="bf16+8"), shapes, torch.float32, 3, none_grad_for=1)
    # gradient clipping: gradients large enough that the clip is active (norms of 4..6 against clip_at = 1)
    run_traj("adamw_clip_l2", A, dict(gradient_clipping="l2_clip_", weight_decay=0.01), shapes, torch.float32, 3, grad_scale=1.0)
    run_traj("laprop_clip_rmsnorm", L, dict(gradient_clipping="rmsnorm_clip_"), shapes, torch.float32, 3, grad_scale=3.0)
    run_traj("adamw_updclip_l2", A, dict(update_clipping="l2_clip_", weight_decay=0.01), shapes, torch.float32, 4)
    run_traj("laprop_updclip_global_rms_caution_ecc", L, dict(update_clipping="global_rmsnorm_clip", caution=True, ecc="bf16+8", lr=0.01),
             shapes, torch.float32, 4)  # fmt: skip
    run_traj("adamw_clip_global_l2_bf16grad", A, dict(gradient_clipping="global_l2norm_clip"), shapes, torch.bfloat16, 3, grad_scale=1.0)
    run_traj("laprop_clip_global_rms_ecc", L, dict(gradient_clipping="global_rmsnorm_clip", ecc="bf16+8"), shapes, torch.float32, 3,
             grad_scale=3.0)  # fmt: skip


def make_variant_trajectories():
    """ADOPT, AdEMAMix and NAdam (heavyball/__init__.py:640-681, :124-164, :83-121) on the same tiny tensors."""
    shapes = [(4, 8), (16,), (3, 5)]
    O, M, N = heavyball.ADOPT, heavyball.AdEMAMix, heavyball.NAdam
    run_traj("adopt_fp32", O, dict(weight_decay=0.01), shapes, torch.float32, 5)
    run_traj("adopt_ecc_caution", O, dict(ecc="bf16+8", caution=True), shapes, torch.bfloat16, 5, grad_scale=1e-3)
    run_traj("adopt_mars_paramecc", O, dict(mars=True, ecc="bf16+16", param_ecc="bf16+8", weight_decay=0.1, cautious_weight_decay=True),
             shapes, torch.float32, 4)  # fmt: skip
    run_traj("adopt_none_grad", O, dict(), shapes, torch.float32, 4, none_grad_for=1)
    run_traj("ademamix_fp32", M, dict(weight_decay=0.01), shapes, torch.float32, 5)
    run_traj("ademamix_warmup_ecc_caution", M, dict(beta3_warmup=10, alpha_warmup=8, ecc="bf16+8", caution=True), shapes, torch.bfloat16, 5,
             grad_scale=1e-3)  # fmt: skip
    run_traj("ademamix_mars_bf16_storage", M, dict(mars=True, storage_dtype="bfloat16", alpha=5.0), shapes, torch.float32, 3)
    run_traj("nadam_fp32", N, dict(weight_decay=0.01), shapes, torch.float32, 5)
    run_traj("nadam_decoupled_ecc_caution", N, dict(weight_decay=0.01, decoupled_weight_decay=True, ecc="bf16+8", caution=True),
             shapes, torch.bfloat16, 5, grad_scale=1e-3)  # fmt: skip
    run_traj("nadam_mars_paramecc", N, dict(mars=True, ecc="bf16+16", param_ecc="bf16+8", momentum_decay=0.1), shapes, torch.float32, 4)


def make_palm_trajectories():
    """``palm=True`` (heavyball/chainable.py:1921-1925, :2693-2694): beta2 = 1 - step ** -beta2_scale, written back into
    the group's betas each step, ahead of the update transform (and of MARS' index in the state keys)."""
    shapes = [(4, 8), (16,), (3, 5)]
    run_traj("adamw_palm", heavyball.AdamW, dict(palm=True, weight_decay=0.01), shapes, torch.float32, 6)
    run_traj("laprop_palm_ecc", heavyball.LaProp, dict(palm=True, beta2_scale=0.6, ecc="bf16+8"), shapes, torch.bfloat16, 5, grad_scale=1e-3)
    run_traj("adamw_palm_mars", heavyball.AdamW, dict(palm=True, mars=True), shapes, torch.float32, 4)
    run_traj("adopt_palm", heavyball.ADOPT, dict(palm=True), shapes, torch.float32, 4)
    run_traj("nadam_palm", heavyball.NAdam, dict(palm=True), shapes, torch.float32, 4)


def make_clip_combinations():
    """Clipping together with the switches it interacts with (heavyball/chainable.py:2676-2701): MARS runs ahead of the
    gradient clip; with update clipping the transform is the un-fused one and the update buffer has the gradient's dtype."""
    shapes = [(4, 8), (16,), (3, 5)]
    A, L = heavyball.AdamW, heavyball.LaProp
    run_traj("adamw_mars_clip_l2", A, dict(mars=True, gradient_clipping="l2_clip_", weight_decay=0.01), shapes, torch.float32, 4, grad_scale=1.0)
    run_traj("laprop_mars_clip_global_rms_ecc_bf16grad", L, dict(mars=True, gradient_clipping="global_rmsnorm_clip", ecc="bf16+8", caution=True),
             shapes, torch.bfloat16, 4, grad_scale=3.0)  # fmt: skip
    run_traj("adamw_updclip_l2_bf16grad", A, dict(update_clipping="l2_clip_", weight_decay=0.01), shapes, torch.bfloat16, 4)
    run_traj("laprop_updclip_rms_mars_bf16grad_ecc", L, dict(update_clipping="rmsnorm_clip_", mars=True, ecc="bf16+8", caution=True, lr=0.01),
             shapes, torch.bfloat16, 4)  # fmt: skip
    run_traj("adopt_updclip_l2", heavyball.ADOPT, dict(update_clipping="l2_clip_", weight_decay=0.01), shapes, torch.float32, 5)
    run_traj("ademamix_updclip_global_l2_ecc", heavyball.AdEMAMix, dict(update_clipping="global_l2norm_clip", ecc="bf16+8"), shapes, torch.float32, 4)
    run_traj("nadam_updclip_rms", heavyball.NAdam, dict(update_clipping="rmsnorm_clip_", weight_decay=0.01), shapes, torch.float32, 4)
    run_traj("nadam_updclip_l2_decoupled_caution", heavyball.NAdam, dict(update_clipping="l2_clip_", weight_decay=0.01, decoupled_weight_decay=True,
                                                                         caution=True), shapes, torch.float32, 4)  # fmt: skip


def make_both_clips():
    """MARS, a gradient clip, an update clip and caution in one chain (heavyball/chainable.py:2693-2701): caution's sign test in the
    chain's tail reads the gradient as MARS left it (heavyball/chainable.py:646), not the raw one."""
    shapes = [(4, 8), (16,), (3, 5)]
    run_traj("adamw_mars_clip_updclip_caution", heavyball.AdamW, dict(mars=True, gradient_clipping="l2_clip_", update_clipping="rmsnorm_clip_",
                                                                      caution=True, weight_decay=0.01, mars_gamma=0.5), shapes, torch.float32, 5,
             grad_scale=1.0)  # fmt: skip
    run_traj("laprop_mars_clip_updclip_caution_bf16grad_ecc", heavyball.LaProp, dict(mars=True, gradient_clipping="global_l2norm_clip",
                                                                                     update_clipping="l2_clip_", caution=True, ecc="bf16+8",
                                                                                     mars_gamma=0.5, lr=0.01), shapes, torch.bfloat16, 5,
             grad_scale=1.0)  # fmt: skip


def make_fp16_unfused():
    """float16 gradients on the un-fused chain (heavyball/chainable.py:2676-2701): the update buffer is float16, every write into
    it (the transform's result, the clip's) is a plain cast, and the tail compares it with the float16 gradient."""
    shapes = [(4, 8), (16,), (3, 5)]
    run_traj("adamw_updclip_l2_fp16grad", heavyball.AdamW, dict(update_clipping="l2_clip_", weight_decay=0.01), shapes, torch.float16, 4)
    run_traj("laprop_updclip_rms_mars_fp16grad_ecc_caution", heavyball.LaProp, dict(update_clipping="rmsnorm_clip_", mars=True, ecc="bf16+8",
                                                                                   caution=True, lr=0.01), shapes, torch.float16, 4)  # fmt: skip
    run_traj("adopt_updclip_global_l2_fp16grad", heavyball.ADOPT, dict(update_clipping="global_l2norm_clip"), shapes, torch.float16, 5)


def make_group_norms():
    """MuonAdamW with clips by a norm over the whole group (heavyball/__init__.py:475-540, heavyball/chainable.py:2696-2701): the clips
    sit around the route, so one norm spans the matrices of the Muon route and the vectors of the Adam route."""
    shapes = [(8, 16), (16,), (24, 8), (4, 3, 6), (5,)]
    run_traj("muonadamw_global_clips_caution", heavyball.MuonAdamW, dict(gradient_clipping="global_l2norm_clip", update_clipping="global_rmsnorm_clip",
                                                                         caution=True, weight_decay=0.01, lr=0.02), shapes, torch.float32, 4,
             grad_scale=1.0)  # fmt: skip
    run_traj("muonadamw_mars_global_rms_gradclip", heavyball.MuonAdamW, dict(mars=True, gradient_clipping="global_rmsnorm_clip", weight_decay=0.01),
             shapes, torch.float32, 4, grad_scale=3.0)  # fmt: skip


def make_muon_narrow_clips():
    """Muon with an update clip under bf16 gradients: the clip writes into the bf16 update buffer (heavyball/utils.py:3226-3232)."""
    shapes = [(8, 16), (16,), (24, 8), (4, 3, 6)]
    run_traj("muon_updclip_l2_bf16grad", heavyball.Muon, dict(update_clipping="l2_clip_", storage_dtype="bfloat16", lr=0.02), shapes,
             torch.bfloat16, 4)  # fmt: skip
    run_traj("muonadamw_updclip_global_rms_bf16grad_ecc", heavyball.MuonAdamW, dict(update_clipping="global_rmsnorm_clip", ecc="bf16+8", lr=0.02),
             shapes, torch.bfloat16, 4)  # fmt: skip


def make_soap_mars_combinations():
    """SOAP with MARS ahead of narrow moments (mars_old_grad is stored like them) and ahead of a gradient clip (the factors are
    initialised from the corrected gradient, the preconditioner sees the clipped one)."""
    shapes = [(8, 16), (16,), (12, 6)]
    run_traj("soap_mars_ecc", heavyball.SOAP, dict(mars=True, ecc="bf16+8", precondition_frequency=3), shapes, torch.float32, 6)
    run_traj("soap_mars_bf16_storage_caution", heavyball.SOAP, dict(mars=True, storage_dtype="bfloat16", caution=True, precondition_frequency=3),
             shapes, torch.float32, 6)  # fmt: skip
    run_traj("soap_mars_clip_global_l2", heavyball.SOAP, dict(mars=True, gradient_clipping="global_l2norm_clip", precondition_frequency=3,
                                                              mars_gamma=0.1), shapes, torch.float32, 6, grad_scale=1.0)  # fmt: skip
    run_traj("soap_mars_clip_rms_caution", heavyball.SOAP, dict(mars=True, gradient_clipping="rmsnorm_clip_", caution=True, precondition_frequency=3),
             shapes, torch.float32, 6, grad_scale=3.0)  # fmt: skip


def make_soap_split_combinations():
    """SOAP with split=True together with the switches that keep state or take norms outside the preconditioner: with split the
    whole chain runs per block (heavyball/utils.py:1612-1623), so MARS' old gradient, caution's count, the per-tensor norms of
    the clips, narrow moments and the ECC pair of the parameter are all per block.  (20, 12) -> six blocks, (16,) -> two vectors,
    (6, 30) -> four blocks."""
    shapes = [(20, 12), (16,), (6, 30)]
    base = dict(split=True, max_precond_dim=8, precondition_frequency=3)
    run_traj("soap_split_caution", heavyball.SOAP, dict(base, caution=True, weight_decay=0.1), shapes, torch.float32, 6)
    run_traj("soap_split_mars", heavyball.SOAP, dict(base, mars=True, mars_gamma=0.1), shapes, torch.float32, 6)
    run_traj("soap_split_ecc", heavyball.SOAP, dict(base, ecc="bf16+8"), shapes, torch.float32, 6)
    run_traj("soap_split_bf16_storage", heavyball.SOAP, dict(base, storage_dtype="bfloat16"), shapes, torch.float32, 6)
    run_traj("soap_split_param_ecc", heavyball.SOAP, dict(base, param_ecc="bf16+8"), shapes, torch.float32, 6)
    run_traj("soap_split_clip_l2", heavyball.SOAP, dict(base, gradient_clipping="l2_clip_"), shapes, torch.float32, 6, grad_scale=1.0)
    run_traj("soap_split_updclip_rms_caution", heavyball.SOAP, dict(base, update_clipping="rmsnorm_clip_", caution=True, lr=0.05), shapes,
             torch.float32, 6)  # fmt: skip


def make_soap_narrow_gradients():
    """SOAP under 16-bit gradients without promote: the preconditioner promotes its input (heavyball/chainable.py:1261), but the
    factors and the eigenbases are created in the gradient's dtype (heavyball/utils.py:1381, :996), the factors are rewritten
    through copy_stochastic_ at every step and the bases at every refresh."""
    shapes = [(8, 16), (16,), (12, 6)]
    run_traj("soap_bf16grad", heavyball.SOAP, dict(precondition_frequency=3), shapes, torch.bfloat16, 6)
    run_traj("soap_fp16grad_caution", heavyball.SOAP, dict(precondition_frequency=3, caution=True), shapes, torch.float16, 6)
    run_traj("soap_bf16grad_mars_clip_l2", heavyball.SOAP, dict(precondition_frequency=3, mars=True, mars_gamma=0.1, gradient_clipping="l2_clip_"),
             shapes, torch.bfloat16, 6, grad_scale=1.0)  # fmt: skip
    run_traj("soap_bf16param", heavyball.SOAP, dict(precondition_frequency=3, weight_decay=0.1), shapes, torch.bfloat16, 6, param_dtype=torch.bfloat16)
    run_traj("soap_bf16grad_split_ecc", heavyball.SOAP, dict(precondition_frequency=3, split=True, max_precond_dim=8, ecc="bf16+8"),
             [(20, 12), (16,), (6, 30)], torch.bfloat16, 6)  # fmt: skip


def make_muon_fp16_gradients():
    """Muon on float16 gradients without promote: the norm, its clamp and the quotient are float16 arithmetic ahead of the bf16
    stochastic round (heavyball/utils.py:555-556), the orthogonalised update goes back to float16 (:577) and is scaled there."""
    shapes = [(8, 16), (16,), (24, 8), (4, 3, 6)]
    run_traj("muon_fp16grad", heavyball.Muon, dict(weight_decay=0.01), shapes, torch.float16, 4)
    run_traj("muon_fp16grad_mars_caution", heavyball.Muon, dict(mars=True, caution=True), shapes, torch.float16, 4)
    run_traj("muonadamw_fp16grad_caution", heavyball.MuonAdamW, dict(caution=True, weight_decay=0.01), shapes, torch.float16, 4)
    run_traj("muon_legacy_fp16grad", heavyball.Muon, dict(), [(16, 16), (16,), (24, 8), (8, 8)], torch.float16, 4, mode="legacy_newtonschulz")
    # clips around the float16 route: both write into a float16 buffer through a plain cast (heavyball/utils.py:2348-2349)
    run_traj("muon_updclip_l2_fp16grad", heavyball.Muon, dict(update_clipping="l2_clip_", lr=0.02), shapes, torch.float16, 4)
    run_traj("muonadamw_clip_l2_updclip_global_rms_fp16grad", heavyball.MuonAdamW,
             dict(gradient_clipping="l2_clip_", update_clipping="global_rmsnorm_clip", lr=0.02), shapes, torch.float16, 4, grad_scale=1.0)
    out = {}
    gen = torch.Generator().manual_seed(13)
    for name, shape in [("sq", (16, 16)), ("wide", (8, 32)), ("tall", (32, 8)), ("sq64", (64, 64))]:
        G = (torch.randn(shape, generator=gen) * 1e-2).half()
        out[f"{name}/G"] = G.clone()
        with half_rounding():
            out[f"{name}/ns5"] = heavyball.utils.zeropower_via_newtonschulz5(G.clone(), 5).clone()
            if shape[0] == shape[1]:
                out[f"{name}/legacy"] = heavyball.utils.legacy_zeropower_via_newtonschulz5(G.clone(), 5).clone()
            tmp = G.clone()
            heavyball.utils.inplace_orthogonal_(tmp, out=tmp, scale_mode="scale")
            out[f"{name}/orthogonal_scaled"] = tmp.clone()
    torch.save(out, os.path.join(HERE, "ns5_fp16.pt"))


def make_more_switches():
    """Muon, MuonAdamW and SOAP under switches beyond their defaults: MARS ahead of the momentum / the preconditioner, clipping
    and ECC on MuonAdamW, SOAP's preconditioner schedule."""
    shapes = [(8, 16), (16,), (24, 8), (4, 3, 6)]
    run_traj("muon_mars", heavyball.Muon, dict(mars=True, weight_decay=0.01), shapes, torch.float32, 4)
    run_traj("muon_mars_ecc_caution", heavyball.Muon, dict(mars=True, ecc="bf16+8", caution=True), shapes, torch.float32, 4)
    run_traj("muon_mars_bf16grad", heavyball.Muon, dict(mars=True, storage_dtype="bfloat16"), shapes, torch.bfloat16, 4)
    run_traj("muonadamw_mars_clip", heavyball.MuonAdamW, dict(mars=True, gradient_clipping="l2_clip_", weight_decay=0.01), shapes, torch.float32,
             4, grad_scale=1.0)  # fmt: skip
    run_traj("muonadamw_ecc_updclip", heavyball.MuonAdamW, dict(ecc="bf16+8", update_clipping="rmsnorm_clip_"), shapes, torch.float32, 4)
    run_traj("muonadamw_plain_ema_bf16_storage", heavyball.MuonAdamW, dict(nesterov=False, storage_dtype="bfloat16"), shapes, torch.float32, 4)
    run_traj("muon_param_ecc_caution", heavyball.Muon, dict(param_ecc="bf16+8", caution=True, weight_decay=0.01), shapes, torch.float32, 4)
    run_traj("muonadamw_param_ecc16_mars", heavyball.MuonAdamW, dict(param_ecc="bf16+16", mars=True), shapes, torch.float32, 4)
    # bf16 gradients: the un-fused scale_by_adam of the vector route writes its result into a bf16 update buffer
    run_traj("muonadamw_bf16grad_ecc_caution", heavyball.MuonAdamW, dict(ecc="bf16+8", caution=True, weight_decay=0.01), shapes, torch.bfloat16, 4)
    soap_shapes = [(8, 16), (16,), (12, 6)]
    run_traj("soap_mars", heavyball.SOAP, dict(mars=True, precondition_frequency=3), soap_shapes, torch.float32, 6)
    # use_precond_schedule=True cannot be recorded: the reference itself fails on it (heavyball/utils.py:2411 calls .clamp on the
    # python int that heavyball/utils.py:3497 hands it)
    # a vector of three elements: its 3 x 3 factor has full rank by the first refresh (one outer product a step), so the refreshed
    # basis is determined by the data and not by the rounding noise that fills the null space of a rank-deficient factor
    run_traj("soap_precondition_1d", heavyball.SOAP, dict(precondition_1d=True, precondition_frequency=3), [(8, 16), (3,), (12, 6)],
             torch.float32, 6)  # fmt: skip
    # switches of SOAP that act outside the preconditioner (the parameter's storage) or on its moments' storage; a combination the
    # reference itself cannot run is reported and leaves no fixture
    for name, kw in [("soap_param_ecc_caution", dict(param_ecc="bf16+8", caution=True, precondition_frequency=3)),
                     ("soap_ecc", dict(ecc="bf16+8", precondition_frequency=3)),
                     ("soap_bf16_storage", dict(storage_dtype="bfloat16", precondition_frequency=3)),
                     ("soap_precond_grad_accum", dict(precond_grad_accum=True, precondition_frequency=3))]:  # fmt: skip
        try:
            run_traj(name, heavyball.SOAP, kw, soap_shapes, torch.float32, 6)
        except Exception as exc:  # noqa: BLE001
            print(f"{name}: the reference fails with {type(exc).__name__}: {str(exc)[:200]}")


def make_ns5():
    """Newton-Schulz vectors straight from the reference's functions, the bf16 stochastic round made round-half-up."""
    out = {}
    gen = torch.Generator().manual_seed(7)
    for name, shape in [("sq", (16, 16)), ("wide", (8, 32)), ("tall", (32, 8)), ("sq64", (64, 64))]:
        G = torch.randn(shape, generator=gen) * 1e-2
        out[f"{name}/G"] = G.clone()
        with half_rounding():
            out[f"{name}/ns5"] = heavyball.utils.zeropower_via_newtonschulz5(G.clone(), 5).clone()
            if shape[0] == shape[1]:
                out[f"{name}/legacy"] = heavyball.utils.legacy_zeropower_via_newtonschulz5(G.clone(), 5).clone()
            tmp = G.clone()
            heavyball.utils.inplace_orthogonal_(tmp, out=tmp, scale_mode="scale")
            out[f"{name}/orthogonal_scaled"] = tmp.clone()
    torch.save(out, os.path.join(HERE, "ns5.pt"))


def make_legacy():
    """zeroth_power_mode = "legacy_newtonschulz": square matrices take the single coefficient triple and its input rounding
    (heavyball/utils.py:637-657, :790-795), with fp32 and with bf16 gradients; Newton-Schulz vectors on bf16 inputs."""
    shapes = [(16, 16), (16,), (24, 8), (8, 8)]
    run_traj("muon_legacy", heavyball.Muon, dict(weight_decay=0.01), shapes, torch.float32, 4, mode="legacy_newtonschulz")
    run_traj("muon_legacy_bf16grad", heavyball.Muon, dict(storage_dtype="bfloat16"), shapes, torch.bfloat16, 4, mode="legacy_newtonschulz")
    out = {}
    gen = torch.Generator().manual_seed(11)
    for name, shape in [("sq", (16, 16)), ("wide", (8, 32)), ("tall", (32, 8)), ("sq64", (64, 64))]:
        G = (torch.randn(shape, generator=gen) * 1e-2).bfloat16()
        out[f"{name}/G"] = G.clone()
        with half_rounding():
            out[f"{name}/ns5"] = heavyball.utils.zeropower_via_newtonschulz5(G.clone(), 5).clone()
            if shape[0] == shape[1]:
                out[f"{name}/legacy"] = heavyball.utils.legacy_zeropower_via_newtonschulz5(G.clone(), 5).clone()
    torch.save(out, os.path.join(HERE, "ns5_bf16.pt"))


def make_polar_express():
    """zeroth_power_mode = "thinky_polar_express": square matrices take the ten-step schedule of msign (heavyball/utils.py:605-631,
    :796-797), the others the default one; a trajectory under fp32 and one under bf16 gradients, and vectors from msign itself."""
    shapes = [(16, 16), (16,), (24, 8), (8, 8)]
    run_traj("muon_polar_express", heavyball.Muon, dict(weight_decay=0.01), shapes, torch.float32, 4, mode="thinky_polar_express")
    run_traj("muon_polar_express_bf16grad_caution", heavyball.Muon, dict(caution=True), shapes, torch.bfloat16, 4, mode="thinky_polar_express")
    out = {}
    gen = torch.Generator().manual_seed(17)
    for name, shape, dt in [("sq", (16, 16), torch.float32), ("sq64", (64, 64), torch.float32), ("sq96", (96, 96), torch.float32),
                            ("sq64_bf16", (64, 64), torch.bfloat16), ("sq64_fp16", (64, 64), torch.float16)]:  # fmt: skip
        G = (torch.randn(shape, generator=gen) * 1e-2).to(dt)
        out[f"{name}/G"] = G.clone()
        with half_rounding():
            out[f"{name}/msign"] = heavyball.utils.msign(G.clone(), 10).clone()
    torch.save(out, os.path.join(HERE, "msign.pt"))


def make_muon():
    shapes = [(8, 16), (16,), (24, 8), (4, 3, 6)]
    run_traj("muon_default", heavyball.Muon, dict(weight_decay=0.01), shapes, torch.float32, 4)
    run_traj("muon_c4", heavyball.Muon, dict(betas=(0.95, 0.99)), shapes, torch.float32, 3)
    # the other three momentum forms of Muon (heavyball/__init__.py:723-737)
    run_traj("muon_plain_ema", heavyball.Muon, dict(nesterov=False, weight_decay=0.01), shapes, torch.float32, 4)
    run_traj("muon_heavyball", heavyball.Muon, dict(nesterov=False, heavyball_momentum=True), shapes, torch.float32, 4)
    run_traj("muon_nesterov_heavyball", heavyball.Muon, dict(nesterov=True, heavyball_momentum=True), shapes, torch.float32, 4)
    run_traj("muon_clip_l2", heavyball.Muon, dict(gradient_clipping="l2_clip_"), shapes, torch.float32, 3, grad_scale=1.0)
    run_traj("muon_ecc", heavyball.Muon, dict(ecc="bf16+8", weight_decay=0.01), shapes, torch.float32, 4)
    run_traj("muon_bf16_storage_bf16_grad", heavyball.Muon, dict(storage_dtype="bfloat16"), shapes, torch.bfloat16, 4)
    run_traj("muon_heavyball_ecc16", heavyball.Muon, dict(ecc="fp16+16", nesterov=False, heavyball_momentum=True), shapes, torch.float32, 3)
    run_traj("muon_updclip_global_rms", heavyball.Muon, dict(update_clipping="global_rmsnorm_clip", lr=0.02), shapes, torch.float32, 3)
    run_traj("muonadamw_default", heavyball.MuonAdamW, dict(weight_decay=0.01), shapes, torch.float32, 4)
    run_traj("muonadamw_caution", heavyball.MuonAdamW, dict(betas=(0.95, 0.999), caution=True, warmup_steps=2), shapes, torch.float32, 3)


def make_soap():
    """SOAP trajectories: list-valued state (Q, GG) is flattened to Q/0, Q/1 ... by run_traj."""
    shapes = [(8, 16), (16,), (12, 6)]
    run_traj("soap_default", heavyball.SOAP, dict(), shapes, torch.float32, 6)
    run_traj("soap_c5", heavyball.SOAP, dict(precondition_frequency=10, shampoo_beta=0.95, max_precond_dim=8192), shapes, torch.float32, 12)
    run_traj("soap_maxdim", heavyball.SOAP, dict(precondition_frequency=3, max_precond_dim=10), shapes, torch.float32, 5)
    run_traj("soap_clip_global_l2", heavyball.SOAP, dict(gradient_clipping="global_l2norm_clip", precondition_frequency=3), shapes, torch.float32,
             5, grad_scale=1.0)  # fmt: skip
    run_traj("soap_updclip_l2", heavyball.SOAP, dict(update_clipping="l2_clip_", precondition_frequency=3), shapes, torch.float32, 5)
    # dimension merging: (12,4,3,3) -> (12,36) and (8,3,6) -> (8,18) with the first setting, (12,4,9) and (8,3,6) with the
    # second. The first refresh comes once the factors have full rank (4 gradients): power iteration + QR on a
    # rank-deficient factor amplifies rounding noise, and such a trajectory pins nothing.
    conv = [(12, 4, 3, 3), (8, 3, 6)]
    run_traj("soap_merge", heavyball.SOAP, dict(precondition_frequency=4, max_precond_dim=64), conv, torch.float32, 6)
    run_traj("soap_merge3d", heavyball.SOAP, dict(precondition_frequency=2, max_precond_dim=12), conv, torch.float32, 5)
    # merge_dims=False: the parameters as they are, one factor per dimension ((12,4,3,3) has four)
    run_traj("soap_no_merge", heavyball.SOAP, dict(merge_dims=False, precondition_frequency=4), conv, torch.float32, 6)
    # split: every dimension above max_precond_dim is cut into blocks, each block preconditioned with a state of its own:
    # (20,12) -> six blocks, (16,) -> two vectors, (6,30) -> four blocks
    run_traj("soap_split", heavyball.SOAP, dict(split=True, max_precond_dim=8, precondition_frequency=3, weight_decay=0.1),
             [(20, 12), (16,), (6, 30)], torch.float32, 6)  # fmt: skip
    # palm: beta2 = 1 - step ** -beta2_scale heads the chain
    run_traj("soap_palm", heavyball.SOAP, dict(palm=True, beta2_scale=0.7, precondition_frequency=3), shapes, torch.float32, 6)


def make_checkpoints():
    """Checkpoints as the reference writes them: ``state_dict()`` after two steps, the parameters at that point, the
    gradients of a third step and the parameters it leads to.  A loader that restores the checkpoint and takes the third
    step has to land on the same parameters."""
    import copy

    shapes = [(4, 8), (16,), (3, 5)]
    cases = [
        ("laprop_ecc", heavyball.LaProp, dict(ecc="bf16+8"), torch.bfloat16, 1e-3),
        ("adamw_mars_caution_ecc_paramecc", heavyball.AdamW, dict(mars=True, caution=True, ecc="bf16+8", param_ecc="bf16+8"), torch.bfloat16, 1e-3),
        ("adamw_fp32_wd", heavyball.AdamW, dict(weight_decay=0.01, warmup_steps=5), torch.float32, 1e-2),
        ("muon", heavyball.Muon, dict(weight_decay=0.01), torch.float32, 1e-2),
        ("soap", heavyball.SOAP, dict(precondition_frequency=2), torch.float32, 1e-2),
        ("adopt", heavyball.ADOPT, dict(weight_decay=0.01), torch.float32, 1e-2),
        ("ademamix_ecc", heavyball.AdEMAMix, dict(ecc="bf16+8", alpha_warmup=5), torch.float32, 1e-2),
        ("nadam_ecc", heavyball.NAdam, dict(ecc="bf16+8", weight_decay=0.01), torch.bfloat16, 1e-3),
    ]
    for name, cls, kwargs, gdt, gscale in cases:
        gen = torch.Generator().manual_seed(0)
        sh = [(8, 16), (16,), (12, 6)] if cls in (heavyball.Muon, heavyball.SOAP) else shapes
        params = [torch.nn.Parameter(torch.randn(s_, generator=gen) * 0.02) for s_ in sh]
        for p in params:
            p.grad_dtype = None
        out = {"meta/kwargs": json.dumps(kwargs), "meta/cls": cls.__name__}
        with half_rounding():
            opt = cls(params, **kwargs)
            for k in range(1, 4):
                g = torch.Generator().manual_seed(2000 + k)
                grads = [(torch.randn(p.shape, generator=g) * gscale).to(gdt) for p in params]
                if k == 3:
                    out["sd"] = copy.deepcopy(opt.state_dict())
                    for i, p in enumerate(params):
                        out[f"p{i}"] = p.detach().clone()
                        out[f"g{i}"] = grads[i].clone()
                for p, gr in zip(params, grads):
                    p.grad = gr.clone()
                opt.step()
            for i, p in enumerate(params):
                out[f"after/p{i}"] = p.detach().clone()
        path = os.path.join(HERE, f"ckpt_{name}.pt")
        torch.save(out, path)
        torch.load(path, weights_only=True)  # the fixture must load without executing anything


if __name__ == "__main__":
    which = sys.argv[1:] or ["layout", "scalars", "ecc", "traj", "variants", "palm", "clipcombo", "bothclips", "fp16unfused", "groupnorms", "muonnarrow", "soapmars", "soapsplit", "soapnarrow", "muonfp16", "polar", "switches", "ns5", "legacy", "muon", "soap", "ckpt"]
    if "layout" in which:
        make_layout()
    if "scalars" in which:
        make_scalars()
    if "ecc" in which:
        make_ecc()
    if "traj" in which:
        make_trajectories()
    if "variants" in which:
        make_variant_trajectories()
    if "palm" in which:
        make_palm_trajectories()
    if "clipcombo" in which:
        make_clip_combinations()
    if "bothclips" in which:
        make_both_clips()
    if "fp16unfused" in which:
        make_fp16_unfused()
    if "groupnorms" in which:
        make_group_norms()
    if "muonnarrow" in which:
        make_muon_narrow_clips()
    if "soapmars" in which:
        make_soap_mars_combinations()
    if "soapsplit" in which:
        make_soap_split_combinations()
    if "soapnarrow" in which:
        make_soap_narrow_gradients()
    if "switches" in which:
        make_more_switches()
    if "ns5" in which:
        make_ns5()
    if "muon" in which:
        make_muon()
    if "legacy" in which:
        make_legacy()
    if "muonfp16" in which:
        make_muon_fp16_gradients()
    if "polar" in which:
        make_polar_express()
    if "soap" in which:
        make_soap()
    if "ckpt" in which:
        make_checkpoints()

"""GPU parity of the fused AdamW / LaProp step, through the C ABI, against (a) the golden trajectories written from the
reference and (b) the CPU oracle on larger seeded inputs.  Everything is compared bit for bit: fp32 parameters and
moments, bf16/fp16 primaries, int8/int16 corrections; stochastic rounding either disabled ("half") or drawn from the
shared Philox stream."""

import glob
import json
import os

import pytest
import torch

import heavyball_amd
from heavyball_amd import _lib
from tests import helpers as H

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
TRAJ = [p for p in sorted(glob.glob(os.path.join(GOLDEN, "traj_*.pt"))) if "muon" not in p and "soap" not in p]
DEV = "cuda:0"
CLS = {"AdamW": (heavyball_amd.AdamW, "adam"), "LaProp": (heavyball_amd.LaProp, "laprop"), "ADOPT": (heavyball_amd.ADOPT, "adopt"),
       "AdEMAMix": (heavyball_amd.AdEMAMix, "ademamix"), "NAdam": (heavyball_amd.NAdam, "nadam")}  # fmt: skip


@pytest.mark.parametrize("path", TRAJ, ids=[os.path.basename(p)[5:-3] for p in TRAJ])
def test_matches_reference_trajectory(path):
    """Same inputs as the fixture, rounding disabled on both sides: every tensor the reference produced must match to
    the stated tolerance (fp32 1e-6 relative, bf16 1 ulp, ECC pairs one correction unit)."""
    d = torch.load(path, weights_only=True)
    print("case", os.path.basename(path), flush=True)
    kwargs = json.loads(d["meta/kwargs"])
    if "betas" in kwargs:
        kwargs["betas"] = tuple(kwargs["betas"])
    cls, _ = CLS[d["meta/cls"]]
    n = len([k for k in d if k.startswith("init/p")])
    params = [torch.nn.Parameter(d[f"init/p{i}"].clone().to(DEV)) for i in range(n)]
    for p in params:
        p.grad_dtype = None
    heavyball_amd.HBOptimizer.rounding = "half"
    try:
        opt = cls(params, **kwargs)
    finally:
        heavyball_amd.HBOptimizer.rounding = "philox"
    opt.rounding = "half"
    none_first = "none_grad" in path
    for k in range(1, d["meta/steps"] + 1):
        for i, p in enumerate(params):
            p.grad = None if (none_first and k == 1 and i == 1) else d[f"step{k}/g{i}"].clone().to(DEV)
        opt.step()
        torch.cuda.synchronize()
        for i, p in enumerate(params):
            prefix = f"step{k}/state{i}/"
            st = opt.state[p].get(0, {}) if p in opt.state else {}
            want = {"param": d[f"step{k}/p{i}"], **{kk[len(prefix):]: d[kk] for kk in d if kk.startswith(prefix)}}
            if "step" in want:
                assert int(st["step"]) == int(want["step"])
            # clipping carries a reduction; ADOPT's momentum spans many orders of magnitude: both compare in the tensor's scale
            check = H.assert_close_in_scale if ("clip" in path or "adopt" in path) else H.assert_close_to_reference
            check({"param": p.data, **st}, want, f"step {k} tensor {i}")
        assert opt.param_groups[0]["step"] is None
        assert opt.param_groups[0]["lr"] == opt.param_groups[0]["base_lr"]


# ragged shapes: sizes that are not multiples of 8 or of the chunk, a tensor of exactly one chunk, one of size 1
RAGGED = [(127, 33), (4096,), (1,), (5, 7, 3), (8193,), (64, 96)]

CASES = [
    ("adamw_fp32_c1", "AdamW", dict(lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01), torch.float32, 1e-2),
    ("laprop_ecc_c2", "LaProp", dict(ecc="bf16+8"), torch.bfloat16, 1e-3),
    ("adamw_c3", "AdamW", dict(mars=True, caution=True, ecc="bf16+8", param_ecc="bf16+8"), torch.bfloat16, 1e-3),
    ("laprop_mars_caution_cwd", "LaProp", dict(mars=True, caution=True, weight_decay=0.1, cautious_weight_decay=True), torch.float32, 1e-2),
    ("adamw_bf16_storage", "AdamW", dict(storage_dtype="bfloat16", weight_decay=0.01), torch.float32, 1e-2),
    ("laprop_fp16_16_paramecc_bf16_16", "LaProp", dict(ecc="fp16+16", param_ecc="bf16+16", mars=True), torch.float32, 1e-2),
    ("adamw_fp16_8_f16grad", "AdamW", dict(ecc="fp16+8", mars=True, caution=True, warmup_steps=2), torch.float16, 1e-2),
    ("adamw_mars_ecc_f32grad", "AdamW", dict(mars=True, ecc="bf16+8", caution=True), torch.float32, 1e-2),
    ("adopt_fp32", "ADOPT", dict(weight_decay=0.01), torch.float32, 1e-2),
    ("adopt_ecc_caution_c2grads", "ADOPT", dict(ecc="bf16+8", caution=True), torch.bfloat16, 1e-3),
    ("adopt_mars_paramecc_cwd", "ADOPT", dict(mars=True, ecc="bf16+16", param_ecc="bf16+8", weight_decay=0.1, cautious_weight_decay=True),
     torch.float32, 1e-2),
    ("ademamix_fp32", "AdEMAMix", dict(weight_decay=0.01), torch.float32, 1e-2),
    ("ademamix_warmup_ecc_caution", "AdEMAMix", dict(beta3_warmup=10, alpha_warmup=3, ecc="bf16+8", caution=True), torch.bfloat16, 1e-3),
    ("ademamix_mars_bf16_storage_paramecc", "AdEMAMix", dict(mars=True, storage_dtype="bfloat16", param_ecc="fp16+16", alpha=5.0),
     torch.float16, 1e-2),
    ("nadam_fp32_coupled_wd", "NAdam", dict(weight_decay=0.01), torch.float32, 1e-2),
    ("nadam_decoupled_ecc_caution", "NAdam", dict(weight_decay=0.01, decoupled_weight_decay=True, ecc="bf16+8", caution=True),
     torch.bfloat16, 1e-3),
    ("nadam_mars_paramecc_coupled_caution", "NAdam", dict(mars=True, ecc="bf16+16", param_ecc="bf16+8", momentum_decay=0.1, weight_decay=0.05,
                                                          caution=True), torch.float32, 1e-2),
    ("nadam_bf16_storage", "NAdam", dict(storage_dtype="bfloat16"), torch.float32, 1e-2),
    # palm: beta2 = 1 - step ** -beta2_scale (heavyball/chainable.py:1921-1925)
    ("adamw_palm", "AdamW", dict(palm=True, weight_decay=0.01), torch.float32, 1e-2),
    ("laprop_palm_ecc_mars", "LaProp", dict(palm=True, beta2_scale=0.6, ecc="bf16+8", mars=True), torch.bfloat16, 1e-3),
    ("adopt_palm", "ADOPT", dict(palm=True), torch.float32, 1e-2),
    ("nadam_palm_caution", "NAdam", dict(palm=True, caution=True), torch.float32, 1e-2),
]


@pytest.mark.parametrize("rounding", ["half", "philox"])
@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_matches_oracle(case, rounding):
    name, cls_name, kwargs, gdt, gscale = case
    print("case", name, rounding, flush=True)
    cls, kind = CLS[cls_name]
    host, params, opt, orc = H.build_pair(cls, kind, RAGGED, kwargs, DEV, rounding=rounding)
    if kwargs.get("param_ecc"):
        H.compare(opt, orc, params, "after construction")
    H.run_steps(opt, orc, params, RAGGED, 4, gdt, gscale, DEV, none_for={2: [1, 3]}, tag=name)


def test_adopt_warmup_is_shared_by_the_tensors_of_a_step():
    """heavyball/chainable.py:597-610: while any tensor of a step still lacks its warm-up, every tensor of that step takes
    the warm-up (exp_avg_sq is set again, no update).  A tensor without a gradient at step 1 delays everyone at step 2."""
    name, cls_name, kwargs, gdt, gscale = "adopt_late_tensor", "ADOPT", dict(ecc="bf16+8"), torch.float32, 1e-2
    cls, kind = CLS[cls_name]
    host, params, opt, orc = H.build_pair(cls, kind, RAGGED, kwargs, DEV)
    before = [p.detach().clone() for p in params]
    H.run_steps(opt, orc, params, RAGGED, 2, gdt, gscale, DEV, none_for={1: [1, 3]}, tag=name)
    assert all(torch.equal(p.detach(), b) for p, b in zip(params, before)), "two warm-up steps must not move the parameters"
    assert [opt.state[p][0]["_warmup_1"] for p in params] == [2, 1, 2, 1, 2, 2]
    H.run_steps(opt, orc, params, RAGGED, 2, gdt, gscale, DEV, tag=name)
    assert not any(torch.equal(p.detach(), b) for p, b in zip(params, before))


@pytest.mark.parametrize("cls_name,kwargs", [("AdamW", dict(weight_decay=0.1)), ("AdamW", dict(storage_dtype="bfloat16", mars=True, caution=True)),
                                             ("LaProp", dict(weight_decay=0.1, caution=True)), ("LaProp", dict(storage_dtype="bfloat16"))],
                         ids=["adamw", "adamw_bf16_moments_mars_caution", "laprop_caution", "laprop_bf16_moments"])
def test_bf16_params_plain(cls_name, kwargs):
    """bf16 parameters without param_ecc: the parameter write is a stochastic round (heavyball/utils.py:2368-2369).  With
    bf16 gradients over fp32 or bf16 moments: the mixed-precision set-ups that have kernels of their own."""
    shapes = [(33, 9), (4100,), (8192 + 40,)]
    cls, kind = CLS[cls_name]
    for rounding in ("half", "philox"):
        gen = torch.Generator().manual_seed(0)
        host = [(torch.randn(s, generator=gen) * 0.02).bfloat16() for s in shapes]
        params = [torch.nn.Parameter(h.clone().to(DEV)) for h in host]
        opt = cls(params, **kwargs)
        opt.rounding, opt.rng_seed = rounding, 5
        from oracle import first_order as fo
        from oracle.rounding import HalfRounding, PhiloxRounding

        r = HalfRounding() if rounding == "half" else PhiloxRounding(5, base=opt._buckets[0][0].slab.offsets_np.tolist())
        orc = fo.FirstOrderOracle(kind, [h.clone() for h in host], rounding=r, **kwargs)
        H.run_steps(opt, orc, params, shapes, 3, torch.bfloat16, 1e-2, DEV, tag="bf16 params " + rounding)


@pytest.mark.parametrize("mars", [False, True], ids=["plain", "mars"])
@pytest.mark.parametrize("rounding", ["half", "philox"])
def test_caution_count_on_updates_that_nearly_cancel(mars, rounding):
    """Caution's count pass decides most signs from the bf16 primaries of exp_avg (and of MARS' old gradient) and loads the
    int8 corrections only where they could matter.  Gradients built from the oracle's own state put every element next to
    the two decisions that can go either way: exp_avg*(1-a1) + g*a1 within +-2^-6 of zero (the corrections reach 2^-9 of
    exp_avg), and the MARS-corrected gradient within +-2^-6 of zero.  The step must stay bit-identical to the oracle's:
    one miscounted element changes the rescale of the whole tensor."""
    from oracle.ecc import EccTensor

    shapes = [(8192 + 24,), (96, 130), (5000,)]
    kwargs = dict(caution=True, ecc="bf16+8", param_ecc="bf16+8", mars=mars)
    host, params, opt, orc = H.build_pair(heavyball_amd.AdamW, "adam", shapes, kwargs, DEV, rounding=rounding)
    H.run_steps(opt, orc, params, shapes, 2, torch.bfloat16, 1e-3, DEV, tag="ordinary steps")
    gen = torch.Generator().manual_seed(5)
    for k in (3, 4, 5):
        a1 = (1 - 0.9) / (1 - 0.9**k)  # 1 - beta_debias(beta1, step)
        c = 0.0025 * 0.9 / (1 - 0.9)  # MARS: g + c * (g - old_g), heavyball/utils.py:3623-3627 as chainable.py:645 calls it
        grads = []
        for i, sh in enumerate(shapes):
            st = orc.state[i]
            key = next(kk for kk in st if kk.endswith("exp_avg_0"))
            m = EccTensor(st[key], st[key + "::ecc"]).decode()
            eps = (torch.rand(sh, generator=gen) * 2 - 1) * 2.0**-6
            target = -m * ((1 - a1) / a1) * (1 + eps)  # the (corrected) gradient that nearly cancels exp_avg
            if mars:
                ok = next(kk for kk in st if "old_grad" in kk and not kk.endswith("::ecc"))
                og = EccTensor(st[ok], st[ok + "::ecc"]).decode()
                g = (target + c * og) / (1 + c)
                zero_gc = og * (c / (1 + c)) * (1 + eps)  # ... and, on a third of the elements, one whose correction nearly cancels itself
                g = torch.where(torch.rand(sh, generator=gen) < 1 / 3, zero_gc, g)
            else:
                g = target
            grads.append(g.to(torch.bfloat16))
        for p_, g_ in zip(params, grads):
            p_.grad = g_.to(DEV)
        opt.step()
        orc.step([g_.clone() for g_ in grads])
        H.compare(opt, orc, params, f"nearly cancelling step {k}")


def _random_case(seed):
    """One draw from the switches the five fused optimizers share, on ragged shapes around the chunk and work-unit sizes."""
    import random

    rnd = random.Random(seed)
    cls_name = rnd.choice(["AdamW", "LaProp", "ADOPT", "AdEMAMix", "NAdam"])
    kwargs = dict(mars=rnd.random() < 0.4, caution=rnd.random() < 0.4)
    if rnd.random() < 0.5:
        kwargs["weight_decay"] = rnd.choice([0.01, 0.1])
        kwargs["cautious_weight_decay"] = rnd.random() < 0.3
    if rnd.random() < 0.3:
        kwargs["warmup_steps"] = rnd.choice([1, 3])
    if rnd.random() < 0.2 and cls_name != "AdEMAMix":
        kwargs["palm"] = True
    storage = rnd.choice(["f32", "bf16", "bf16+8", "bf16+8", "bf16+16", "fp16+8", "fp16+16"])
    if "+" in storage:
        kwargs["ecc"] = storage
    elif storage == "bf16":
        kwargs["storage_dtype"] = "bfloat16"
    gdt = rnd.choice([torch.float32, torch.bfloat16, torch.bfloat16, torch.float16])
    bf16_params = False
    pe = rnd.choice([None, None, "bf16+8", "fp16+16", "bf16+16"])
    if pe is not None:
        kwargs["param_ecc"] = pe
    elif gdt == torch.bfloat16 and rnd.random() < 0.4:
        bf16_params = True
    if cls_name == "NAdam" and rnd.random() < 0.5:
        kwargs["decoupled_weight_decay"] = True
    sizes = [1, 7, 8, 9, 255, 256, 257, 1023, 1024, 2047, 2048, 2049, 4095, 4096, 4097, 6143, 8191, 8192, 8193, 12345]
    shapes = [(rnd.choice(sizes),) for _ in range(rnd.randint(2, 5))] + [(rnd.randint(1, 70), rnd.randint(1, 90))]
    rnd.shuffle(shapes)
    none_for = {2: [rnd.randrange(len(shapes))]} if rnd.random() < 0.3 else None
    return cls_name, kwargs, gdt, bf16_params, shapes, none_for, rnd.choice(["half", "philox"])


@pytest.mark.parametrize("seed", range(600))
def test_random_configurations_match_oracle(seed):
    """Seeded draws over optimizer, switches, storage formats, gradient and parameter dtypes and ragged sizes (one element up
    to three chunks, around every multiple of the work unit), three steps each, bit for bit against the oracle: the
    combinations nobody listed by hand, most of them on the kernel that switches on run-time format codes."""
    from oracle import first_order as fo
    from oracle.rounding import HalfRounding, PhiloxRounding

    cls_name, kwargs, gdt, bf16_params, shapes, none_for, rounding = _random_case(seed)
    print("case", seed, cls_name, kwargs, gdt, "bf16 params" if bf16_params else "", shapes, none_for, rounding, flush=True)
    cls, kind = CLS[cls_name]
    if not bf16_params:
        host, params, opt, orc = H.build_pair(cls, kind, shapes, kwargs, DEV, rounding=rounding)
    else:
        gen = torch.Generator().manual_seed(0)
        host = [(torch.randn(s, generator=gen) * 0.02).bfloat16() for s in shapes]
        params = [torch.nn.Parameter(h.clone().to(DEV)) for h in host]
        opt = cls(params, **kwargs)
        opt.rounding, opt.rng_seed = rounding, 77
        r = HalfRounding() if rounding == "half" else PhiloxRounding(77, base=opt._buckets[0][0].slab.offsets_np.tolist())
        orc = fo.FirstOrderOracle(kind, [h.clone() for h in host], rounding=r, **kwargs)
    H.run_steps(opt, orc, params, shapes, 3, gdt, 1e-2 if gdt == torch.float32 else 1e-3, DEV, none_for=none_for, tag=f"draw {seed}")


def test_c1_full_size():
    """Benchmark configuration 1 at its full size: 4 fp32 tensors, 9,438,208 elements, 10 steps, bit-exact against the oracle."""
    shapes = [(1024, 1024), (1024,), (4096, 1024), (1024, 4096)]
    kwargs = dict(lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01)
    host, params, opt, orc = H.build_pair(heavyball_amd.AdamW, "adam", shapes, kwargs, DEV)
    H.run_steps(opt, orc, params, shapes, 10, torch.float32, 1e-2, DEV, check_each=False, tag="C1")


def test_c2_slice_philox():
    """Benchmark configuration 2 on one transformer layer plus a truncated embedding (7.9M elements), shared Philox stream."""
    shapes = [(768, 2304), (2304,), (768, 768), (768,), (768, 3072), (3072,), (3072, 768), (768,), (768,), (768,), (768,), (768,), (1031, 768)]
    host, params, opt, orc = H.build_pair(heavyball_amd.LaProp, "laprop", shapes, dict(ecc="bf16+8"), DEV)
    H.run_steps(opt, orc, params, shapes, 3, torch.bfloat16, 1e-3, DEV, check_each=False, tag="C2 slice")


def test_c3_slice_philox():
    """Benchmark configuration 3 on a reduced layer (same roles and dtypes), shared Philox stream, 5 steps."""
    shapes = [(512, 512), (128, 512), (1792, 512), (512, 1792), (512,), (1003, 512)]
    kwargs = dict(mars=True, caution=True, ecc="bf16+8", param_ecc="bf16+8")
    host, params, opt, orc = H.build_pair(heavyball_amd.AdamW, "adam", shapes, kwargs, DEV)
    H.run_steps(opt, orc, params, shapes, 5, torch.bfloat16, 1e-3, DEV, check_each=False, tag="C3 slice")


def test_mars_write_grad():
    shapes = [(37, 5), (4099,)]
    host, params, opt, orc = H.build_pair(heavyball_amd.AdamW, "adam", shapes, dict(mars=True), DEV)
    opt.mars_write_grad = True
    grads = H.make_grads(shapes, 1, torch.bfloat16, 1e-2)
    dev_grads = [g.to(DEV) for g in grads]
    for p, g in zip(params, dev_grads):
        p.grad = g
    opt.step()
    cpu = [g.clone() for g in grads]
    orc.step(cpu)  # the oracle overwrites its gradient list in place, as the reference does
    for i in range(len(shapes)):
        H.assert_bit_equal(dev_grads[i], cpu[i], f"corrected gradient {i}")


def test_state_dict_roundtrip_continues_identically():
    """save -> load into a fresh optimizer -> both continue bit-identically (test/test_save_restore.py:51-75)."""
    shapes = [(65, 17), (300,)]
    kwargs = dict(mars=True, caution=True, ecc="bf16+8", param_ecc="bf16+8")
    host, params, opt, orc = H.build_pair(heavyball_amd.AdamW, "adam", shapes, kwargs, DEV, rounding="half")
    H.run_steps(opt, orc, params, shapes, 2, torch.bfloat16, 1e-3, DEV, tag="before save")
    sd = opt.state_dict()
    import io

    buf = io.BytesIO()
    torch.save(sd, buf)
    buf.seek(0)
    sd2 = torch.load(buf, weights_only=True)
    params2 = [torch.nn.Parameter(p.detach().clone()) for p in params]
    for p in params2:
        p.grad_dtype = None
    opt2 = heavyball_amd.AdamW(params2, **kwargs)
    opt2.rounding, opt2.rng_seed = "half", opt.rng_seed
    # parameters are bf16 already, so the constructor left the corrections at zero; the checkpoint restores them
    opt2.load_state_dict(sd2)
    for k in (3, 4):
        grads = H.make_grads(shapes, k, torch.bfloat16, 1e-3)
        for plist, o in ((params, opt), (params2, opt2)):
            for p, g in zip(plist, grads):
                p.grad = g.to(DEV)
            o.step()
    for a, b in zip(params, params2):
        H.assert_bit_equal(a.data, b.data, "param after resume")
        for key, v in opt.state[a][0].items():
            if isinstance(v, torch.Tensor) and key != "step":
                H.assert_bit_equal(opt2.state[b][0][key], v, key)
        assert opt2.state[b][0]["update_by_adam_exp_avg_0"].dtype == torch.bfloat16
        assert opt2.state[b][0]["update_by_adam_exp_avg_0::ecc"].dtype == torch.int8


@pytest.mark.parametrize("rounding", ["half", "philox"])
def test_param_groups_step_independently(rounding):
    """Two parameter groups with their own lr, betas and weight decay, one of them without gradients at step 2, and a third
    group added after construction: every group keeps its own step counter (heavyball/chainable.py:2531-2570), so each
    behaves like an optimizer of its own over the steps in which it had gradients.  Bit for bit against one oracle per group."""
    from oracle import first_order as fo
    from oracle.rounding import HalfRounding, PhiloxRounding

    shapes = [[(130, 33), (4100,)], [(8193,)], [(77,), (5, 9)]]
    common = dict(ecc="bf16+8", caution=True)
    per_group = [dict(lr=1e-3, weight_decay=0.1), dict(lr=3e-3, betas=(0.8, 0.95)), dict(lr=2e-3, mars=True, weight_decay=0.01)]
    gen = torch.Generator().manual_seed(4)
    host = [[torch.randn(s, generator=gen) * 0.02 for s in grp] for grp in shapes]
    params = [[torch.nn.Parameter(h.clone().to(DEV)) for h in grp] for grp in host]
    for grp in params:
        for p in grp:
            p.grad_dtype = None
    opt = heavyball_amd.AdamW([dict(params=params[0], **per_group[0]), dict(params=params[1], **per_group[1])], **common)
    opt.rounding, opt.rng_seed = rounding, 9
    opt.add_param_group(dict(params=params[2], **per_group[2]))
    assert len(opt.param_groups) == 3 and opt.param_groups[2]["ecc"] == "bf16+8" and opt.param_groups[2]["mars"] is True
    oracles = []
    for gi in range(3):
        base = opt._buckets[gi][0].slab.offsets_np.tolist() if gi in opt._buckets else None
        r = HalfRounding() if rounding == "half" else None
        oracles.append([fo, host[gi], {**common, **per_group[gi]}, r, base])
    built = {}
    for k in range(1, 5):
        for gi in range(3):
            has_grads = not (gi == 1 and k == 2)
            grads = H.make_grads(shapes[gi], 10 * gi + k, torch.bfloat16, 1e-3) if has_grads else [None] * len(shapes[gi])
            for p, g in zip(params[gi], grads):
                p.grad = None if g is None else g.to(DEV)
            oracles[gi].append(grads)
        opt.step()
        torch.cuda.synchronize()
        for gi in range(3):
            if gi not in built:  # the slab offsets (the noise generator's index base) exist once the group has stepped
                _, h, kw, r, _ = oracles[gi][:5]
                if r is None:
                    r = PhiloxRounding(9, base=opt._buckets[gi][0].slab.offsets_np.tolist())
                built[gi] = fo.FirstOrderOracle("adam", [t.clone() for t in h], rounding=r, **kw)
            grads = oracles[gi][-1]
            if any(g is not None for g in grads):
                built[gi].step([None if g is None else g.clone() for g in grads])
            H.compare(opt, built[gi], params[gi], f"group {gi} step {k}")
    steps = [int(opt.state[grp[0]][0]["step"]) for grp in params]
    assert steps == [4, 3, 4], steps


def test_error_paths():
    L = _lib.lib()
    d = _lib.HbStepDesc()
    assert L.hb_fused_step(d, None) != 0
    assert b"offsets" in L.hb_last_error() or b"required" in L.hb_last_error()
    p = [torch.nn.Parameter(torch.zeros(4, device=DEV))]
    opt = heavyball_amd.AdamW(p)
    p[0].grad = torch.zeros(4, device=DEV)
    opt.rounding = "bogus"  # makes the step raise after the group's lr/step were set (chainable.py:2567-2570 restores them)
    with pytest.raises(ValueError):
        opt.step()
    assert opt.param_groups[0]["step"] is None and opt.param_groups[0]["lr"] == opt.param_groups[0]["base_lr"]
    opt.rounding = "half"
    p[0].grad = torch.ones(4, device=DEV)
    opt.step()
    assert int(opt.state[p[0]][0]["step"]) == 2


@pytest.mark.parametrize("kind", ["l2_clip_", "rmsnorm_clip_", "global_l2norm_clip", "global_rmsnorm_clip"])
@pytest.mark.parametrize("grad_dtype", [torch.float32, torch.bfloat16])
def test_gradient_clipping_matches_oracle(kind, grad_dtype):
    """gradient_clipping through step(): gather, per-tensor reduction, scale, bf16 re-rounding, then the fused step, on
    ragged shapes with the clip active (norms of 10..500 against clip_at = 1).  The norms are summed in a different order
    than ATen's, so the scale can differ in its last bit: fp32 gradients agree to 2e-6 of each tensor's scale instead of
    bit for bit.  With bf16 gradients that last bit can move an element across a stochastic-rounding threshold (chance
    2^-16 per element), which shifts that element's clipped gradient by one bf16 ulp: there a handful of elements
    (<= 1e-3 of them over three steps) may sit outside the bar, by at most the 2^-8 such a flip can cause."""
    print("case", kind, grad_dtype, flush=True)
    kwargs = dict(gradient_clipping=kind, weight_decay=0.01)
    host, params, opt, orc = H.build_pair(heavyball_amd.LaProp, "laprop", RAGGED, kwargs, DEV, rounding="philox")
    for p in params:
        p.grad_dtype = None
    for k in range(1, 4):
        grads = H.make_grads(RAGGED, k, grad_dtype, 1.0)
        for p, g in zip(params, grads):
            p.grad = g.to(DEV)
        opt.step()
        orc.step([g.clone() for g in grads])
        torch.cuda.synchronize()
        for i, p in enumerate(params):
            st = opt.state[p][0]
            want = {"param": orc.params[i], **{kk: v for kk, v in orc.state[i].items() if kk != "step"}}
            if grad_dtype == torch.float32:
                H.assert_close_in_scale({"param": p.data, **st}, want, f"{kind} step {k} tensor {i}")
                continue
            for key, w in want.items():
                g = (p.data if key == "param" else st[key]).detach().cpu()
                off = (g - w).abs() > 2e-6 * (w.abs() + w.abs().max())
                assert int(off.sum()) <= max(4, int(1e-3 * w.numel())), (kind, k, i, key, int(off.sum()))
                assert ((g - w).abs() <= 2.0**-7 * (w.abs() + w.abs().max())).all(), (kind, k, i, key)


CLIP_COMBOS = [
    # (name, class, kwargs, gradient dtype, gradient scale)
    ("adamw_mars_gradclip_l2", "AdamW", dict(mars=True, gradient_clipping="l2_clip_", weight_decay=0.01), torch.float32, 1.0),
    ("laprop_mars_gradclip_global_rms_ecc_caution", "LaProp", dict(mars=True, gradient_clipping="global_rmsnorm_clip", ecc="bf16+8", caution=True),
     torch.bfloat16, 3.0),
    ("nadam_mars_gradclip_rms_paramecc", "NAdam", dict(mars=True, gradient_clipping="rmsnorm_clip_", param_ecc="bf16+8", ecc="bf16+16"),
     torch.float32, 2.0),
    ("adamw_updclip_l2_bf16grad", "AdamW", dict(update_clipping="l2_clip_", weight_decay=0.01), torch.bfloat16, 1e-2),
    ("laprop_updclip_rms_mars_ecc_caution_bf16grad", "LaProp", dict(update_clipping="rmsnorm_clip_", mars=True, ecc="bf16+8", caution=True, lr=0.01),
     torch.bfloat16, 1e-2),
    ("adopt_updclip_l2", "ADOPT", dict(update_clipping="l2_clip_", weight_decay=0.01), torch.float32, 1e-2),
    ("ademamix_updclip_global_l2_ecc", "AdEMAMix", dict(update_clipping="global_l2norm_clip", ecc="bf16+8"), torch.float32, 1e-2),
    ("nadam_updclip_rms_coupled_wd", "NAdam", dict(update_clipping="rmsnorm_clip_", weight_decay=0.01), torch.float32, 1e-2),
    ("nadam_updclip_l2_decoupled_caution_bf16grad", "NAdam", dict(update_clipping="l2_clip_", weight_decay=0.01, decoupled_weight_decay=True,
                                                                  caution=True), torch.bfloat16, 1e-2),
    # float16 gradients: the update buffer is float16, written by plain casts
    ("adamw_updclip_l2_fp16grad", "AdamW", dict(update_clipping="l2_clip_", weight_decay=0.01), torch.float16, 1e-2),
    ("laprop_updclip_rms_mars_ecc_caution_fp16grad", "LaProp", dict(update_clipping="rmsnorm_clip_", mars=True, ecc="bf16+8", caution=True, lr=0.01),
     torch.float16, 1e-2),
    ("adopt_updclip_global_l2_fp16grad", "ADOPT", dict(update_clipping="global_l2norm_clip"), torch.float16, 1e-2),
    # MARS, both clips and caution in one chain: the tail's sign test reads the MARS-corrected gradient
    ("adamw_mars_both_clips_caution", "AdamW", dict(mars=True, gradient_clipping="l2_clip_", update_clipping="rmsnorm_clip_", caution=True,
                                                    weight_decay=0.01, mars_gamma=0.5), torch.float32, 1.0),
    ("laprop_mars_both_clips_caution_bf16grad_ecc", "LaProp", dict(mars=True, gradient_clipping="global_l2norm_clip", update_clipping="l2_clip_",
                                                                   caution=True, ecc="bf16+8", mars_gamma=0.5, lr=0.01), torch.bfloat16, 1.0),
    # float16 gradients under a gradient clip: the clipped values return to the float16 buffer through a cast
    ("adamw_gradclip_rms_fp16grad", "AdamW", dict(gradient_clipping="rmsnorm_clip_", weight_decay=0.01), torch.float16, 1.0),
    ("laprop_mars_gradclip_l2_fp16grad_ecc", "LaProp", dict(mars=True, gradient_clipping="l2_clip_", ecc="bf16+8", mars_gamma=0.5), torch.float16, 1.0),
    # gradients of several dtypes in one bucket (a tuple: dealt out to the tensors in turn): every clip and rounding is per tensor
    ("adamw_gradclip_global_l2_mixed_grads", "AdamW", dict(gradient_clipping="global_l2norm_clip", weight_decay=0.01),
     (torch.float32, torch.bfloat16, torch.float16), 1.0),
    ("laprop_mars_both_clips_caution_mixed_grads", "LaProp", dict(mars=True, gradient_clipping="rmsnorm_clip_", update_clipping="global_rmsnorm_clip",
                                                                  caution=True, mars_gamma=0.5, lr=0.01), (torch.bfloat16, torch.float32), 1.0),
    ("adopt_updclip_l2_mixed_grads_ecc", "ADOPT", dict(update_clipping="l2_clip_", ecc="bf16+8"), (torch.float16, torch.float32, torch.bfloat16), 1e-2),
]


@pytest.mark.parametrize("case", CLIP_COMBOS, ids=[c[0] for c in CLIP_COMBOS])
def test_clipping_combinations_match_oracle(case):
    """Clipping together with the switches it interacts with (heavyball/chainable.py:2676-2701): MARS ahead of the gradient
    clip (a pass of its own, then the step without MARS on the clipped slab); update clipping on every fused optimizer (the
    step kernel in update-only mode, the clip, then the parameter update) and with bf16 gradients, where the update is
    rounded to bf16 after the transform and again after the clip, as the reference's update buffer is.  The norms are
    summed in a different order than ATen's, hence agreement to 2e-6 of each tensor's scale (bf16 updates: one ulp more
    where the last bit of the scale moves an element across a rounding threshold)."""
    name, cls_name, kwargs, gdt, gscale = case
    print("case", name, flush=True)
    cls, kind = CLS[cls_name]
    host, params, opt, orc = H.build_pair(cls, kind, RAGGED, kwargs, DEV, rounding="philox")
    gdts = [gdt[i % len(gdt)] for i in range(len(RAGGED))] if isinstance(gdt, tuple) else [gdt] * len(RAGGED)
    gdt = torch.bfloat16 if isinstance(gdt, tuple) else gdt  # mixed: the tolerance of the narrowest
    bf16_update = gdt in (torch.bfloat16, torch.float16) and "update_clipping" in kwargs  # a 16-bit update buffer
    for k in range(1, 5):
        grads = [g.to(t) for g, t in zip(H.make_grads(RAGGED, k, torch.float32, gscale), gdts)]
        for p, g in zip(params, grads):
            p.grad = g.to(DEV)
        opt.step()
        orc.step([g.clone() for g in grads])
        torch.cuda.synchronize()
        for i, p in enumerate(params):
            st = opt.state[p][0]
            pw = orc.params[i]
            want = {"param": pw.primary if hasattr(pw, "primary") else pw,
                    **{kk: v for kk, v in orc.state[i].items() if kk != "step" and isinstance(v, torch.Tensor)}}
            got = {"param": p.data, **st}
            if not (bf16_update or gdt in (torch.bfloat16, torch.float16)):
                H.assert_close_in_scale(got, want, f"{name} step {k} tensor {i}")
                continue
            for key, w in want.items():
                if key.endswith("::ecc") or w.dim() == 0:
                    continue
                ck = "param::ecc" if key == "param" else key + "::ecc"
                g_, w_ = got[key].detach().cpu(), w
                if ck in want:
                    from oracle.ecc import EccTensor

                    g_, w_ = EccTensor(g_, got[ck].detach().cpu()).decode(), EccTensor(w_, want[ck]).decode()
                g_, w_ = g_.float(), w_.float()
                off = (g_ - w_).abs() > 2e-6 * (w_.abs() + w_.abs().max()) + (2.0**-8 * w_.abs() if w.dtype != torch.float32 or ck in want else 0)
                assert int(off.sum()) <= max(4, int(2e-3 * w_.numel())), (name, k, i, key, int(off.sum()))
                assert ((g_ - w_).abs() <= 2.0**-6 * (w_.abs() + w_.abs().max())).all(), (name, k, i, key)


def test_unknown_clip_name_raises():
    p = [torch.nn.Parameter(torch.zeros(8, device=DEV))]
    with pytest.raises(ValueError):
        heavyball_amd.AdamW(p, gradient_clipping="no_such_clip")


def test_empty_tensors_and_steps_without_gradients():
    """A zero-sized parameter takes no room in the slab and no workgroup; a step in which no parameter has a gradient
    changes nothing and does not advance the step counter; a parameter whose gradient stays None keeps no state."""
    shapes = [(0,), (5, 3), (0, 7), (4097,)]
    host, params, opt, orc = H.build_pair(heavyball_amd.AdamW, "adam", shapes, dict(weight_decay=0.01, ecc="bf16+8"), DEV)
    before = [p.detach().clone() for p in params]
    opt.step()  # nothing has a gradient
    orc.step([None] * len(shapes))
    torch.cuda.synchronize()
    assert all(torch.equal(p.detach(), b) for p, b in zip(params, before))
    assert all("step" not in (opt.state[p].get(0, {}) if p in opt.state else {}) for p in params)
    H.run_steps(opt, orc, params, shapes, 3, torch.float32, 1e-2, DEV, none_for={1: [1], 2: [3]}, tag="empty")
    assert int(opt.state[params[0]][0]["step"]) == 3 if 0 in opt.state.get(params[0], {}) else True
    assert params[0].numel() == 0 and params[2].numel() == 0


LAYOUT_CASES = [
    ("AdamW", "AdamW", {}, torch.float32),
    ("AdamW_mars", "AdamW", {"mars": True}, torch.float32),
    ("AdamW_ecc", "AdamW", {"ecc": "bf16+8"}, torch.float32),
    ("AdamW_mars_caution_ecc_paramecc", "AdamW", {"mars": True, "caution": True, "ecc": "bf16+8", "param_ecc": "bf16+8"}, torch.bfloat16),
    ("LaProp", "LaProp", {}, torch.float32),
    ("LaProp_ecc", "LaProp", {"ecc": "bf16+8"}, torch.float32),
    ("LaProp_bf16_storage", "LaProp", {"storage_dtype": "bfloat16"}, torch.float32),
    ("Muon", "Muon", {}, torch.float32),
    ("SOAP", "SOAP", {}, torch.float32),
    ("MuonAdamW", "MuonAdamW", {}, torch.float32),
    ("ADOPT", "ADOPT", {}, torch.float32),
    ("ADOPT_mars_ecc", "ADOPT", {"mars": True, "ecc": "bf16+8"}, torch.float32),
    ("AdEMAMix", "AdEMAMix", {}, torch.float32),
    ("AdEMAMix_ecc", "AdEMAMix", {"ecc": "bf16+8"}, torch.float32),
    ("NAdam", "NAdam", {}, torch.float32),
    ("NAdam_ecc", "NAdam", {"ecc": "bf16+8"}, torch.float32),
]


@pytest.mark.parametrize("case", LAYOUT_CASES, ids=[c[0] for c in LAYOUT_CASES])
def test_state_dict_layout_matches_reference(case):
    """state_dict() after two steps: same state keys, dtypes, shapes, is_initialized sets, param-group keys and values,
    "heavyball" sub-dict keys as the reference wrote into tests/golden/layout.json; and it loads with weights_only=True."""
    import io

    name, cls_name, kw, gdt = case
    want = json.load(open(os.path.join(GOLDEN, "layout.json")))[name]
    torch.manual_seed(0)
    params = [torch.nn.Parameter(torch.randn(8, 16, device=DEV)), torch.nn.Parameter(torch.randn(16, device=DEV))]
    opt = getattr(heavyball_amd, cls_name)(params, **kw)
    for _ in range(2):
        for p in params:
            p.grad = (torch.randn(p.shape, device=DEV) * 1e-2).to(p.dtype)
        opt.step()
    torch.cuda.synchronize()
    assert all(p.grad is None for p in params) == want["grad_is_none_after_step"]
    assert [str(p.dtype) for p in params] == want["param_dtypes"]
    sd = opt.state_dict()
    assert sorted(sd["param_groups"][0].keys()) == want["param_group_keys"]
    for k, v in want["param_group_values"].items():
        got = sd["param_groups"][0][k]
        if k == "prev_lr":
            assert isinstance(got, torch.Tensor) and got.dtype == torch.float32 and got.dim() == 0
            continue
        assert (repr(got) == v) if isinstance(v, str) and not isinstance(got, str) else (got == v), (k, got, v)
    assert sorted(sd["heavyball"].keys()) == want["heavyball_keys"]
    for pi, views in want["state_keys"].items():
        for view, entries in views.items():
            got = sd["state"][int(pi)][int(view)]
            assert set(got.keys()) == set(entries.keys()), (set(got.keys()) ^ set(entries.keys()))
            for key, spec in entries.items():
                if isinstance(spec, dict):
                    assert str(got[key].dtype) == spec["dtype"] and list(got[key].shape) == spec["shape"], key
                elif isinstance(spec, list):  # SOAP's Q / GG: one tensor or None per dimension
                    assert len(got[key]) == len(spec), key
                    for t, sp in zip(got[key], spec):
                        if isinstance(sp, dict):
                            assert str(t.dtype) == sp["dtype"] and list(t.shape) == sp["shape"], key
                        else:
                            assert repr(t) == sp, key
                elif key == "is_initialized":
                    assert repr(sorted(got[key])) == spec
    buf = io.BytesIO()
    torch.save(sd, buf)
    buf.seek(0)
    torch.load(buf, weights_only=True)


def test_parameter_rebound_after_construction_is_moved_back_into_the_slab():
    """``p.data`` pointed at fresh storage after the optimizer was built (a swap of averaged weights, ``p.data = ...``):
    the next step must act on the new values and leave the result in ``p``, not in an orphaned slab copy."""
    shapes = [(64, 96), (96,), (1000, 33)]
    host, params, opt, orc = H.build_pair(heavyball_amd.AdamW, "adam", shapes, dict(weight_decay=0.01), DEV, rounding="half")
    H.run_steps(opt, orc, params, shapes, 2, torch.float32, 1e-2, DEV, tag="before")
    homes = [p.data_ptr() for p in params]
    gen = torch.Generator().manual_seed(99)
    fresh = [torch.randn(s, generator=gen) * 0.05 for s in shapes]
    for i in (0, 2):
        params[i].data = fresh[i].to(DEV)  # new storage
        orc.params[i].copy_(fresh[i])
        assert params[i].data_ptr() != homes[i]
    for k in (3, 4):
        grads = H.make_grads(shapes, k, torch.float32, 1e-2)
        for p, g in zip(params, grads):
            p.grad = g.to(DEV)
        opt.step()
        orc.step([g.clone() for g in grads])
        H.compare(opt, orc, params, f"after rebinding, step {k}")
    assert [p.data_ptr() for p in params] == homes
    # a dtype change cannot be absorbed: the slab holds fp32
    params[1].data = params[1].data.bfloat16()
    params[1].grad = torch.zeros(shapes[1], device=DEV)
    with pytest.raises(_lib.HbError, match="dtype"):
        opt.step()


PLAN_CASES = [
    ("laprop_ecc_bf16grad", heavyball_amd.LaProp, dict(ecc="bf16+8"), torch.bfloat16, 1e-3),
    ("adamw_mars_caution_ecc_paramecc", heavyball_amd.AdamW, dict(mars=True, caution=True, ecc="bf16+8", param_ecc="bf16+8", weight_decay=0.01),
     torch.bfloat16, 1e-3),
    ("adamw_fp32_warmup_decay", heavyball_amd.AdamW, dict(weight_decay=0.1, warmup_steps=3, betas=(0.9, 0.999)), torch.float32, 1e-2),
]  # fmt: skip


@pytest.fixture(params=["cpp_loop", "python_loop"])
def tensor_loop(request):
    """The cached-plan step walks its tensors in the C++ helper when that is built, else in Python: both are run."""
    from heavyball_amd import optim

    assert optim.hostloop() is not None, "heavyball_amd/_hostloop.so has not been built"
    before = optim._hostloop_module
    if request.param == "python_loop":
        optim._hostloop_module = None
    yield request.param
    optim._hostloop_module = before


@pytest.mark.parametrize("case", PLAN_CASES, ids=[c[0] for c in PLAN_CASES])
def test_cached_plan_steps_equal_the_general_path(case, tensor_loop):
    """``FirstOrder._fast_step`` replays the launches of the step before with new scalars and gradient pointers.  Two optimizers
    on the same inputs, one with the cached plan switched off, stay bit-identical through ordinary steps and through everything
    that must send a step back to the general path: a missing gradient, a changed learning rate and betas (which the plan reads
    afresh), a gradient of another dtype, a non-contiguous gradient, a parameter rebound to new storage, gradients kept
    (consume_grad=False), a second param group.  The steps the plan took are counted."""
    _, cls, kwargs, gdt, gscale = case
    shapes = [(64, 96), (96,), (1000, 33), (7,)]
    gen = torch.Generator().manual_seed(0)
    host = [torch.randn(s, generator=gen) * 0.02 for s in shapes]
    opts, sets = [], []
    for planned in (True, False):
        params = [torch.nn.Parameter(h.clone().to(DEV)) for h in host]
        for p in params:
            p.grad_dtype = None
        opt = cls([dict(params=params[:3]), dict(params=params[3:], lr=1e-3)], **kwargs)
        opt.rng_seed = 4321
        if not planned:
            opt._plannable = False
        opts.append(opt)
        sets.append(params)
    taken = []
    fast = opts[0]._fast_step
    opts[0]._fast_step = lambda gi, group: (taken.append(gi) if (ok := fast(gi, group)) else None, ok)[1]

    def grads_for(k, dtype=gdt):
        g = torch.Generator().manual_seed(1000 + k)
        return [(torch.randn(s, generator=g) * gscale).to(dtype) for s in shapes]

    def step_both(k, grads):
        for opt, params in zip(opts, sets):
            for p, g in zip(params, grads):
                p.grad = None if g is None else g.to(DEV)
            opt.step()
        torch.cuda.synchronize()
        for i, (p, q) in enumerate(zip(*sets)):
            H.assert_bit_equal(p.data, q.data, f"step {k} param {i}")
            sp, sq = opts[0].state[p].get(0, {}), opts[1].state[q].get(0, {})
            assert set(sp) == set(sq)
            for key, val in sp.items():
                if isinstance(val, torch.Tensor):
                    H.assert_bit_equal(val, sq[key], f"step {k} tensor {i} {key}")

    for k in (1, 2, 3, 4):
        step_both(k, grads_for(k))
    # group 1 replays from its second step on; group 0 rebuilds its plan once more when group 1's state entries have appeared
    assert taken.count(1) == 3 and taken.count(0) >= 2
    taken.clear()
    g5 = grads_for(5)
    g5[1] = None
    step_both(5, g5)  # a tensor without a gradient: the general path, for group 0 only
    assert taken == [1]
    step_both(6, grads_for(6))
    for opt in opts:
        opt.param_groups[0]["lr"] = 5e-4
        opt.param_groups[0]["betas"] = (0.8, 0.95)
        opt.param_groups[1]["weight_decay"] = 0.05
    taken.clear()
    import warnings

    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        step_both(7, grads_for(7))
    assert sorted(taken) == [0, 1]  # new hyper-parameters do not need the general path
    other = torch.float32 if gdt == torch.bfloat16 else torch.bfloat16
    taken.clear()
    step_both(8, grads_for(8, other))  # another gradient dtype: general path, and a new plan from there
    step_both(9, grads_for(9, other))
    assert sorted(taken) == [0, 1]
    step_both(10, grads_for(10))
    g11 = grads_for(11)
    g11[0] = g11[0].t().contiguous().t()  # same values, column-major
    taken.clear()
    step_both(11, g11)
    assert taken == [1]
    for params in sets:
        params[2].data = params[2].data.clone()  # new storage
    step_both(12, grads_for(12))
    step_both(13, grads_for(13))
    for opt in opts:
        opt.consume_grad = False
    taken.clear()
    step_both(14, grads_for(14))
    assert sorted(taken) == [0, 1] and all(p.grad is not None for p in sets[0])
    sd = opts[0].state_dict()
    opts[0].load_state_dict(sd)  # drops the plans; the tensors of the state move, the values stay
    taken.clear()
    step_both(15, grads_for(15))
    assert taken == []
    step_both(16, grads_for(16))
    assert sorted(taken) == [0, 1]


def test_dropped_state_entry_starts_from_zero_again():
    """``del optimizer.state[p]`` for one parameter between steps: its moments restart from zero (the reference's zero_guard
    builds them anew), the other parameters carry on, and ``state_dict()`` lists the rebuilt entries."""
    shapes = [(64, 96), (96,), (1000, 33)]
    host, params, opt, orc = H.build_pair(heavyball_amd.LaProp, "laprop", shapes, dict(ecc="bf16+8"), DEV, rounding="philox")
    H.run_steps(opt, orc, params, shapes, 3, torch.bfloat16, 1e-3, DEV, tag="before")
    del opt.state[params[1]]
    orc.state[1] = {}
    for k in (4, 5):
        grads = H.make_grads(shapes, k, torch.bfloat16, 1e-3)
        for p, g in zip(params, grads):
            p.grad = g.to(DEV)
        opt.step()
        orc.step([g.clone() for g in grads])
        H.compare(opt, orc, params, f"after the drop, step {k}")
    assert "update_by_laprop_exp_avg_0" in opt.state_dict()["state"][1][0]

"""Checkpoint compatibility: a ``state_dict()`` written by the reference (tests/golden/ckpt_*.pt: the state after two steps, the
parameters at that point, the gradients of a third step and the parameters it leads to) is loaded into the optimizer here,
which then takes the third step on the GPU.  The result has to match the reference's to the tolerance of the path
(fp32 8 ulps, ECC pairs one correction unit, Newton-Schulz 2e-2 of the step, SOAP 2e-3 of the step)."""

import glob
import json
import os

import pytest
import torch

import heavyball_amd
from tests import helpers as H

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
DEV = torch.device("cuda:0")
PATHS = sorted(glob.glob(os.path.join(GOLDEN, "ckpt_*.pt")))


def rel_fro(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm().clamp(min=1e-30)).item()


@pytest.mark.parametrize("path", PATHS, ids=[os.path.basename(p)[5:-3] for p in PATHS])
def test_reference_checkpoint_loads_and_continues(path):
    d = torch.load(path, weights_only=True)
    print("case", os.path.basename(path), flush=True)
    kwargs = json.loads(d["meta/kwargs"])
    cls = getattr(heavyball_amd, d["meta/cls"])
    n = len([k for k in d if k.startswith("after/p")])
    pecc = kwargs.get("param_ecc")
    # a fresh model: fp32 parameters with arbitrary values; under param_ecc the optimizer narrows them at construction
    params = [torch.nn.Parameter(torch.zeros(d[f"p{i}"].shape, device=DEV)) for i in range(n)]
    for p in params:
        p.grad_dtype = None
    opt = cls(params, **kwargs)
    opt.rounding = "half"
    # restore the model's parameters (what a model.load_state_dict would do), then the optimizer
    for i, p in enumerate(params):
        assert p.dtype == d[f"p{i}"].dtype, "param_ecc keeps the live parameter in the narrow dtype"
        p.data.copy_(d[f"p{i}"].to(DEV))
    opt.load_state_dict(d["sd"])
    st0 = opt.state[params[0]][0]
    assert int(st0["step"]) == 2
    for key, val in d["sd"]["state"][0][0].items():
        if isinstance(val, torch.Tensor) and key != "step":
            assert st0[key].dtype == val.dtype and torch.equal(st0[key].cpu(), val), key  # storage dtypes restored, values intact
    if pecc:
        assert "param::ecc" in st0 and st0["param::ecc"].dtype == torch.int8
    for i, p in enumerate(params):
        p.grad = d[f"g{i}"].clone().to(DEV)
    opt.step()
    torch.cuda.synchronize()
    assert int(opt.state[params[0]][0]["step"]) == 3
    for i, p in enumerate(params):
        got, want, prev = p.detach().cpu(), d[f"after/p{i}"], d[f"p{i}"]
        if d["meta/cls"] == "Muon" and want.dim() >= 2:
            assert rel_fro(got - prev, want - prev) < 2e-2, i
        elif d["meta/cls"] == "SOAP" and want.dim() >= 2:
            assert rel_fro(got - prev, want - prev) < 2e-3, i
        elif pecc:
            corr = opt.state[p][0]["param::ecc"].cpu()
            # the reference's parameter after the step is a bf16 primary; compare primaries to one bf16 ulp
            assert H.ulp_distance(got, want).max() <= 1, i
            assert corr.dtype == torch.int8
        else:
            assert H.ulp_distance(got, want).max() <= H.FP32_ULPS, (i, int(H.ulp_distance(got, want).max()))
    # and the state dict written here loads back into a second instance
    sd = opt.state_dict()
    params2 = [torch.nn.Parameter(p.detach().clone()) for p in params]
    opt2 = cls(params2, **kwargs)
    opt2.load_state_dict(sd)
    assert int(opt2.state[params2[0]][0]["step"]) == 3


def test_own_checkpoints_for_the_reference_are_current(tmp_path):
    """tests/golden/own_ckpt_*.pt are this implementation's ``state_dict()``s that tests/golden/check_own_checkpoints.py loads
    into the reference (own_ckpt_check.json holds the outcome: every case continues to the same parameters).  They have to be
    what the present code writes: regenerate them and compare every tensor bit for bit."""
    import importlib.util

    spec = importlib.util.spec_from_file_location("write_own_checkpoints", os.path.join(GOLDEN, "write_own_checkpoints.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    mod.main(str(tmp_path))
    with open(os.path.join(GOLDEN, "own_ckpt_check.json")) as f:
        checked = json.load(f)

    def same(a, b, where):
        if isinstance(a, torch.Tensor):
            assert isinstance(b, torch.Tensor) and a.dtype == b.dtype and a.shape == b.shape, where
            assert torch.equal(a.reshape(-1).view(torch.uint8), b.reshape(-1).view(torch.uint8)), where
        elif isinstance(a, dict):
            assert isinstance(b, dict) and set(a) == set(b), (where, sorted(map(str, a)), sorted(map(str, b)))
            for k in a:
                same(a[k], b[k], f"{where}/{k}")
        elif isinstance(a, (list, tuple)):
            assert len(a) == len(b), where
            for i, (x, y) in enumerate(zip(a, b)):
                same(x, y, f"{where}[{i}]")
        else:
            assert a == b, (where, a, b)

    for name, *_ in mod.CASES:
        print("case", name, flush=True)
        assert name in checked, f"{name} has not been loaded into the reference (run tests/golden/check_own_checkpoints.py)"
        new = torch.load(os.path.join(str(tmp_path), f"own_ckpt_{name}.pt"), weights_only=True)
        old = torch.load(os.path.join(GOLDEN, f"own_ckpt_{name}.pt"), weights_only=True)
        same(new, old, name)

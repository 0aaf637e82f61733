"""Loads the checkpoints written by write_own_checkpoints.py into the REFERENCE's optimizers and continues training.

Run in the build container, where the reference tree is mounted at /root/reference:

    python tests/golden/check_own_checkpoints.py

For every own_ckpt_*.pt: the reference's optimizer is constructed on the stored parameters, ``load_state_dict`` takes the
``state_dict()`` this implementation wrote (heavyball/utils.py:1542-1549, heavyball/chainable.py:2452-2484 restore the
"heavyball" entry and the ECC storage dtypes), the third step runs on the CPU with rounding disabled, and the parameters
are compared with the ones this implementation reached on the GPU from the same state: fp32 within 8 ulps, an ECC pair
within one correction unit, the Muon step within 2e-2 and the SOAP step within 5e-3 relative Frobenius (the bars of the
parity tests).  Writes own_ckpt_check.json with the measured deviations.
"""

import glob
import json
import os
import sys

os.environ["TORCH_COMPILE_DISABLE"] = "1"
HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, "/root/reference")
sys.path.insert(1, ROOT)

import torch  # noqa: E402

import heavyball  # noqa: E402
import heavyball.utils  # noqa: E402

from make_golden import half_rounding  # noqa: E402  (same directory: the patch of rand_like / randint_like)
from tests import helpers as H  # noqa: E402

heavyball.utils.compile_mode = None
torch.set_num_threads(1)


def rel_fro(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm().clamp(min=1e-30)).item()


def main():
    report = {}
    for path in sorted(glob.glob(os.path.join(HERE, "own_ckpt_*.pt"))):
        name = os.path.basename(path)[len("own_ckpt_") : -3]
        d = torch.load(path, weights_only=True)
        kwargs = json.loads(d["meta/kwargs"])
        cls = getattr(heavyball, d["meta/cls"])
        n = len([k for k in d if k.startswith("after/p")])
        # the model's parameters come back from the model's own checkpoint; under param_ecc they are the narrow primaries,
        # which the constructor narrows again (exactly) before load_state_dict brings the corrections
        params = [torch.nn.Parameter(d[f"p{i}"].clone().float() if kwargs.get("param_ecc") else d[f"p{i}"].clone()) for i in range(n)]
        for p in params:
            p.grad_dtype = None
        with half_rounding():
            opt = cls(params, **kwargs)
            opt.load_state_dict(d["sd"])
            for i, p in enumerate(params):
                assert torch.equal(p.detach().float(), d[f"p{i}"].float()), "parameters changed by load_state_dict"
                p.grad = d[f"g{i}"].clone()
            st0 = opt.state_(params[0])
            assert int(st0["step"]) == 2
            opt.step()
        entry = {}
        for i, p in enumerate(params):
            want = d[f"after/p{i}"]
            assert p.dtype == want.dtype, (name, i, p.dtype, want.dtype)
            if d["meta/cls"] in ("Muon", "SOAP"):
                step_ref, step_own = p.detach() - d[f"p{i}"], want - d[f"p{i}"]
                err = rel_fro(step_own, step_ref)
                bar = 2e-2 if d["meta/cls"] == "Muon" else 5e-3
                assert err < bar, (name, i, err)
                entry[f"p{i}"] = {"step_rel_fro": err, "bar": bar}
                continue
            got = {"param": want}
            ref = {"param": p.detach()}
            if kwargs.get("param_ecc"):
                # compare the decoded pair: the correction this implementation holds after the step is not in the file (it lives
                # in the state_dict of the step after), so the primaries are compared to one bf16 ulp
                dist = H.ulp_distance(want, p.detach())
                assert dist.max() <= 1, (name, i, int(dist.max()))
                entry[f"p{i}"] = {"max_primary_ulps": int(dist.max())}
                continue
            H.assert_close_to_reference(got, ref, f"{name} p{i}")
            entry[f"p{i}"] = {"max_fp32_ulps": int(H.ulp_distance(want, p.detach()).max())}
        report[name] = entry
        print(name, json.dumps(entry), flush=True)
    with open(os.path.join(HERE, "own_ckpt_check.json"), "w") as f:
        json.dump(report, f, indent=1, sort_keys=True)
    print("all checkpoints of this implementation load into the reference and continue to the same parameters")


if __name__ == "__main__":
    main()

"""Writes checkpoints of THIS implementation for the reference to load (the other direction of ckpt_*.pt).

Run on a machine with an MI355X, from the repository root:

    python tests/golden/write_own_checkpoints.py [output directory, default tests/golden]

For every case: two steps on seeded inputs with rounding disabled, then ``state_dict()``, the parameters at that point,
the gradients of a third step and the parameters that step leads to HERE.  ``check_own_checkpoints.py`` (build container,
where the reference is mounted) loads each ``state_dict`` into the reference's optimizer, takes the third step on the CPU
and compares.  The files hold tensors, strings and plain containers only and load with ``weights_only=True``.
"""

import copy
import json
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import heavyball_amd  # noqa: E402

CASES = [
    # name, class, kwargs, gradient dtype, gradient scale, matrix shapes?
    ("laprop_ecc", "LaProp", dict(ecc="bf16+8"), "bfloat16", 1e-3, False),
    ("adamw_mars_caution_ecc_paramecc", "AdamW", dict(mars=True, caution=True, ecc="bf16+8", param_ecc="bf16+8"), "bfloat16", 1e-3, False),
    ("adamw_fp32_wd", "AdamW", dict(weight_decay=0.01, warmup_steps=5), "float32", 1e-2, False),
    ("muon", "Muon", dict(weight_decay=0.01), "float32", 1e-2, True),
    ("soap", "SOAP", dict(precondition_frequency=2), "float32", 1e-2, True),
    ("adopt", "ADOPT", dict(weight_decay=0.01), "float32", 1e-2, False),
    ("ademamix_ecc", "AdEMAMix", dict(ecc="bf16+8", alpha_warmup=5), "float32", 1e-2, False),
    ("nadam_ecc", "NAdam", dict(ecc="bf16+8", weight_decay=0.01), "bfloat16", 1e-3, False),
]


def to_cpu(x):
    if isinstance(x, torch.Tensor):
        return x.detach().cpu().clone()
    if isinstance(x, dict):
        return {k: to_cpu(v) for k, v in x.items()}
    if isinstance(x, (list, tuple)):
        return type(x)(to_cpu(v) for v in x)
    return x


def main(out_dir):
    dev = torch.device("cuda:0")
    os.makedirs(out_dir, exist_ok=True)
    for name, cls_name, kwargs, gdt, gscale, matrices in CASES:
        gen = torch.Generator().manual_seed(0)
        shapes = [(8, 16), (16,), (12, 6)] if matrices else [(4, 8), (16,), (3, 5)]
        params = [torch.nn.Parameter((torch.randn(s, generator=gen) * 0.02).to(dev)) for s in shapes]
        for p in params:
            p.grad_dtype = None
        heavyball_amd.HBOptimizer.rounding = "half"  # param_ecc encodes at construction
        try:
            opt = getattr(heavyball_amd, cls_name)(params, **kwargs)
        finally:
            heavyball_amd.HBOptimizer.rounding = "philox"
        opt.rounding = "half"
        out = {"meta/kwargs": json.dumps(kwargs), "meta/cls": cls_name}
        for k in range(1, 4):
            g = torch.Generator().manual_seed(2000 + k)
            grads = [(torch.randn(p.shape, generator=g) * gscale).to(getattr(torch, gdt)) for p in params]
            if k == 3:
                torch.cuda.synchronize()
                out["sd"] = to_cpu(copy.deepcopy(opt.state_dict()))
                for i, p in enumerate(params):
                    out[f"p{i}"] = p.detach().cpu().clone()
                    out[f"g{i}"] = grads[i].clone()
            for p, gr in zip(params, grads):
                p.grad = gr.to(dev)
            opt.step()
        torch.cuda.synchronize()
        for i, p in enumerate(params):
            out[f"after/p{i}"] = p.detach().cpu().clone()
        path = os.path.join(out_dir, f"own_ckpt_{name}.pt")
        torch.save(out, path)
        torch.load(path, weights_only=True)  # must load without executing anything
        print("wrote", path, flush=True)


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else os.path.dirname(os.path.abspath(__file__)))

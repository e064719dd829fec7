"""Writes tests/golden/ref_scan_golden.npz from the reference's own tree scan.

Run once, in the development container, where the reference checkout is
mounted at /root/reference:

    python tests/golden/make_golden.py

The only thing about the oracle (oracle/ref_scan.py) that neither the
sequential fp64 recurrence nor closed forms can pin is the bit pattern of the
fp32 tree association order, so those bits are recorded here from
accelerated_scan/ref.py (pure torch, CPU).  The file holds inputs and outputs
only.  Inputs come from seeded torch CPU generators and are stored too, so the
tests do not depend on torch's generator staying stable.
"""

import importlib.util
import math
import sys
from pathlib import Path

import numpy as np
import torch

REFERENCE = Path("/root/reference/accelerated_scan/ref.py")
OUT = Path(__file__).resolve().parent / "ref_scan_golden.npz"


def load_reference():
    spec = importlib.util.spec_from_file_location("reference_ref", REFERENCE)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def main():
    ref = load_reference()
    data = {}

    def real_case(name, seed, shape, reverse=False, grads=False, long_memory=False):
        gen = torch.Generator().manual_seed(seed)
        gates = torch.rand(*shape, generator=gen)
        if long_memory:
            gates = 0.999 + 0.001 * gates
        tokens = torch.rand(*shape, generator=gen)
        data[f"{name}.gates"] = gates.numpy().copy()
        data[f"{name}.tokens"] = tokens.numpy().copy()
        data[f"{name}.reverse"] = np.array(int(reverse))
        if grads:
            gates.requires_grad_(True)
            tokens.requires_grad_(True)
            out = ref.scan(gates, tokens, reverse=reverse)
            grad_out = torch.randn(*shape, generator=gen)
            dg, dt = torch.autograd.grad(out, (gates, tokens), grad_out)
            data[f"{name}.grad_out"] = grad_out.numpy().copy()
            data[f"{name}.d_gates"] = dg.numpy().copy()
            data[f"{name}.d_tokens"] = dt.numpy().copy()
            out = out.detach()
        else:
            with torch.inference_mode():
                out = ref.scan(gates, tokens, reverse=reverse)
        data[f"{name}.out"] = out.numpy().copy()

    # The smallest benchmark configuration: fp32 (1, 64, 1024), U(0,1) gates and tokens.
    real_case("cfg1_fwd", 3407, (1, 64, 1024))
    real_case("pow2_rev", 4, (2, 3, 256), reverse=True)
    real_case("pad_fwd", 42, (2, 3, 1000))            # padded to 1024 with (1, 0)
    real_case("pad_rev", 57, (1, 5, 37), reverse=True)
    real_case("tiny_T2", 5, (1, 2, 2))
    real_case("tiny_T3", 6, (1, 2, 3))
    real_case("long_memory", 7, (1, 4, 4096), long_memory=True)
    real_case("grads_fwd", 8, (2, 4, 300), grads=True)
    real_case("grads_pow2", 9, (1, 4, 512), grads=True)

    # complex gates, real and complex tokens (tests/tests_eq_complex.py:26-47 style inputs)
    gen = torch.Generator().manual_seed(11)
    shape = (1, 4, 600)
    angle = 2 * math.pi * torch.rand(*shape, generator=gen)
    radius = 0.99 + 0.01 * torch.rand(*shape, generator=gen)
    forget = torch.polar(radius, angle).to(torch.complex64)
    real_inputs = torch.randn(*shape, generator=gen).tanh()
    cplx_inputs = torch.complex(torch.randn(*shape, generator=gen), torch.randn(*shape, generator=gen))
    grad_out = torch.complex(torch.randn(*shape, generator=gen), torch.randn(*shape, generator=gen))
    for name, inputs in (("complex_real_tokens", real_inputs), ("complex_complex_tokens", cplx_inputs)):
        f = forget.clone().requires_grad_(True)
        i = inputs.clone().requires_grad_(True)
        out = ref.scan(f, i)
        df, di = torch.autograd.grad(out, (f, i), grad_out)
        data[f"{name}.gates"] = forget.numpy().copy()
        data[f"{name}.tokens"] = inputs.numpy().copy()
        data[f"{name}.grad_out"] = grad_out.numpy().copy()
        data[f"{name}.out"] = out.detach().numpy().copy()
        data[f"{name}.d_gates"] = df.numpy().copy()
        data[f"{name}.d_tokens"] = di.numpy().copy()

    np.savez_compressed(OUT, **data)
    print(f"wrote {OUT} ({OUT.stat().st_size} bytes, {len(data)} arrays, torch {torch.__version__})")


if __name__ == "__main__":
    sys.exit(main())

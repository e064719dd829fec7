"""Max-abs error of the HIP scan against the fp64 recurrence for U(0,1) inputs,
T = 32..65536, shape (1, 512, T) -- the quantity the reference plots in
max-abs-error.png (README.md:60-64 of the reference).  Also reports the torch
tree scan run in the same storage dtype, which is what the reference's kernels
are judged by.  One JSON line per T into FILE (or stdout).

    python tests/precision_table.py [FILE]

A measurement script, not a pytest module: it needs the GPU and uses the
oracle (oracle/seqscan, oracle/ref_scan) as the checker.
"""

import json
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent
for p in (ROOT, ROOT / "accelerated-scan_amd"):
    if str(p) not in sys.path:
        sys.path.insert(0, str(p))


def main(path=None):
    import numpy as np
    import torch

    from accelerated_scan.warp import scan_forward
    from oracle import ref_scan, seqscan

    out = open(path, "w") if path else sys.stdout
    try:
        for T in [2 ** i for i in range(5, 17)]:
            gen = torch.Generator().manual_seed(3407)
            gates32 = torch.rand(1, 512, T, generator=gen)
            tokens32 = torch.rand(1, 512, T, generator=gen)
            rec = {"T": T}
            for name, dt in (("fp32", torch.float32), ("fp16", torch.float16), ("bf16", torch.bfloat16)):
                g = gates32.to(dt)
                x = tokens32.to(dt)
                truth = seqscan.forward(g.float().numpy(), x.float().numpy())
                hip = scan_forward(g.to("cuda:0"), x.to("cuda:0")).float().cpu().numpy()
                tree = ref_scan.scan(g.to("cuda:0"), x.to("cuda:0")).float().cpu().numpy()
                rec[f"{name}_hip_max_abs_err"] = float(np.abs(hip - truth).max())
                rec[f"{name}_tree_scan_same_dtype_max_abs_err"] = float(np.abs(tree - truth).max())
            out.write(json.dumps(rec) + "\n")
            out.flush()
    finally:
        if path:
            out.close()
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1] if len(sys.argv) > 1 else None))

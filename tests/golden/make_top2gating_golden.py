"""Writes tests/golden/top2gating_*.npz: input/output vectors of the reference's own top2gating
(rtp/module/top2gate.py:43-105), the one routine whose order-of-operation details (count-before-drop,
dispatch = combine.bool(), eps clamp) no stock torch layer pins.

Run in the build container only (needs the reference tree on disk):
    python tests/golden/make_top2gating_golden.py /root/reference
The Gumbel sample the reference draws internally is recorded by re-seeding torch's global CPU generator
and drawing it once more with the reference's own gumbel_rsample, so the fixture carries
(logits, noise) -> (l_aux, combine_weights, dispatch_mask).
"""
import os
import sys

import numpy as np
import torch


def main(ref_root: str) -> None:
    sys.path.insert(0, ref_root)
    from rtp.module import top2gate as ref  # noqa: E402  (namespace package: the reference has no __init__.py)

    here = os.path.dirname(os.path.abspath(__file__))
    cpu = torch.device("cpu")
    for name, S, E, seed, scale in [("s16_e4", 16, 4, 1, 1.0), ("s64_e8", 64, 8, 2, 1.0), ("s32_e2", 32, 2, 3, 1.0),
                                    ("s64_e4_skewed", 64, 4, 4, 1.0)]:
        torch.manual_seed(seed)
        logits = torch.randn(S, E) * scale
        if "skewed" in name:
            logits[:, 0] += 2.5  # most tokens pick expert 0 first: exercises the capacity drop
        torch.manual_seed(seed + 1000)
        noise = ref.gumbel_rsample(logits.shape, cpu).clone()
        torch.manual_seed(seed + 1000)
        l_aux, combine, dispatch = ref.top2gating(logits.clone())
        np.savez_compressed(os.path.join(here, f"top2gating_{name}.npz"), logits=logits.numpy(), noise=noise.numpy(),
                            l_aux=l_aux.numpy(), combine_weights=combine.numpy(), dispatch_mask=dispatch.numpy())
        print(name, "l_aux", float(l_aux), "dropped pairs", int(2 * S - dispatch.sum()))


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")

"""Writes tests/golden/mta_golden.npz: small regression vectors for the MTA forward path.

    python tests/golden/make_golden.py

The reference repository ships no golden vectors, known-answer tests or fixtures for this
path (it has no tests at all), and its code was read, not run.  These vectors are
therefore produced by the oracle (oracle/mta_oracle.py) AFTER it has been pinned by the
closed forms, library routines and brute-force C loops of tests/test_oracle.py.  They
guard against drift (a different torch build, an edit to the oracle) and give the GPU
tests fixed inputs and outputs that do not depend on the oracle at run time.
All arrays are float32; inputs are seeded draws.
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import mta_oracle as O  # noqa: E402


def main():
    out = {}
    g = torch.Generator().manual_seed(2024)
    # depthwise causal conv, 6x11, one plane pair
    x = torch.tril(torch.randn(1, 2, 24, 24, generator=g))
    w = 0.2 * torch.randn(2, 6, 11, generator=g)
    out["conv_x"], out["conv_w"] = x.numpy(), w.numpy()
    out["conv_y_causal"] = O.depthwise_conv(x, w, True).numpy()
    out["conv_y_full"] = O.depthwise_conv(x, w, False).numpy()
    # head mixing, dense 4x4, both fills
    hx = torch.randn(1, 4, 12, 12, generator=g)
    hw = torch.eye(4) + 0.1 * torch.randn(4, 4, generator=g)
    out["hm_x"], out["hm_w"] = hx.numpy(), hw.numpy()
    out["hm_y_zero"] = O.head_linear(hx, hw, True, 0.0).numpy()
    out["hm_y_neginf"] = O.head_linear(hx, hw, True, float("-inf")).numpy()
    # full MTA forward, BASELINE config 1 scaled down: B1 H4 S32 D16, 3x5 conv, groups of 2
    q, k, v = O.seeded_qkv(1, 4, 32, 16, torch.float32)
    w_pre = O.seeded_conv_weight(4, 3, 5, 0.1, torch.float32)
    w_post = O.seeded_conv_weight(4, 3, 3, 0.05, torch.float32, seed=77)
    wpsm = O.block_diag_head_weight(4, 2, 0.1, g)
    wposm = O.block_diag_head_weight(4, 2, 0.1, g)
    out.update(mta_q=q.numpy(), mta_k=k.numpy(), mta_v=v.numpy(), mta_w_pre=w_pre.numpy(), mta_w_post=w_post.numpy(),
               mta_wpsm=wpsm.numpy(), mta_wposm=wposm.numpy())
    out["mta_out"] = O.mta_forward(q, k, v, w_pre.unsqueeze(1), wpsm, w_post.unsqueeze(1), wposm).numpy()
    # fused conv attention: B1 H2 S48 D64, 6x11
    cq, ck, cv = O.seeded_qkv(1, 2, 48, 64, torch.float32, seed=42)
    cw = O.seeded_conv_weight(2, 6, 11, 0.05, torch.float32)
    out.update(ca_q=cq.numpy(), ca_k=ck.numpy(), ca_v=cv.numpy(), ca_w=cw.numpy())
    out["ca_out_causal"] = O.conv_attention_forward(cq, ck, cv, cw, True, None).numpy()
    out["ca_out_full"] = O.conv_attention_forward(cq, ck, cv, cw, False, None).numpy()
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "mta_golden.npz")
    np.savez_compressed(path, **{k_: np.asarray(v_, dtype=np.float32) for k_, v_ in out.items()})
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()

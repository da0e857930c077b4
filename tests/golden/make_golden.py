"""Writes the golden fixtures under tests/golden/ from the CPU oracle's float64 closed forms.

The reference holds no stored vectors for this path (its attention tests compare two live
implementations on GPUs), and its packages cannot be imported here, so these vectors are made
by oracle/attn_oracle.py, which tests/test_oracle.py pins independently (brute force, torch's
own CPU attention ops, merge identities).  Run from the repository root:
    python tests/golden/make_golden.py
Inputs are regenerated from seeds at test time; only expected outputs (and tiny inputs) are stored.
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import attn_oracle as O  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def tiny_cases():
    """Brute-force (math.fsum) cases: inputs and outputs stored in full."""
    out = {}
    g = torch.Generator().manual_seed(7)
    for n, (Sq, Sk, D) in enumerate([(1, 1, 4), (3, 8, 4), (8, 3, 8), (17, 17, 8), (5, 33, 8)]):
        q = torch.randn(Sq, D, generator=g, dtype=torch.float64)
        k = torch.randn(Sk, D, generator=g, dtype=torch.float64)
        v = torch.randn(Sk, D, generator=g, dtype=torch.float64)
        scale = D ** -0.5
        o, l = O.attn_bruteforce(q.tolist(), k.tolist(), v.tolist(), scale)
        out[f"t{n}_q"], out[f"t{n}_k"], out[f"t{n}_v"] = q.numpy(), k.numpy(), v.numpy()
        out[f"t{n}_out"], out[f"t{n}_lse"] = np.array(o), np.array(l)
    return out


def probe_rows(S, n, seed):
    g = torch.Generator().manual_seed(seed)
    rows = torch.randperm(S, generator=g)[:n].sort().values
    # always include the first and last row (tile edges)
    rows[0], rows[-1] = 0, S - 1
    return rows


def main():
    np.savez_compressed(os.path.join(HERE, "tiny_bruteforce.npz"), **tiny_cases())

    # C1 PixArt (fp32, full shape): every 37th row of out + the full lse
    c1 = O.make_config("c1_pixart512")
    o, l = O.attn_fwd_ref(c1["q"], c1["k"], c1["v"], 72 ** -0.5)
    np.savez_compressed(os.path.join(HERE, "c1_pixart512.npz"),
                        out_rows=o[:, :, ::37].numpy().astype(np.float32), lse=l.numpy().astype(np.float32))

    # C2 Flux-1024 (bf16 inputs): 64 probe rows x all heads against the full K/V
    c2 = O.make_config("c2_flux1024")
    rows = probe_rows(4608, 64, 2)
    o, l = O.attn_rows_ref(c2["q"], c2["k"], c2["v"], rows)
    np.savez_compressed(os.path.join(HERE, "c2_flux1024_rows.npz"), rows=rows.numpy(),
                        out=o.numpy().astype(np.float32), lse=l.numpy().astype(np.float32))

    # C5-like fp8 case at a CPU-sized sequence (S=2048): reference = fp64 attention of the
    # dequantised inputs
    c5 = O.make_config("c5_wan720p_shard_fp8", S=2048)
    dq = O.dequant(c5["q"], c5["q_descale"])
    dk = O.dequant(c5["k"], c5["k_descale"])
    dv = O.dequant(c5["v"], c5["v_descale"])
    rows = probe_rows(2048, 64, 5)
    o, l = O.attn_rows_ref(dq, dk, dv, rows)
    np.savez_compressed(os.path.join(HERE, "c5_fp8_s2048_rows.npz"), rows=rows.numpy(),
                        out=o.numpy().astype(np.float32), lse=l.numpy().astype(np.float32),
                        q_descale=c5["q_descale"].numpy(), k_descale=c5["k_descale"].numpy(),
                        v_descale=c5["v_descale"].numpy(),
                        q_bytes_head0_row0=c5["q"].view(torch.uint8)[0, 0, 0].numpy())

    # merge: random partials and the float64 fold
    g = torch.Generator().manual_seed(11)
    out = torch.randn(2, 3, 40, 16, generator=g, dtype=torch.float64)
    lse = torch.randn(2, 3, 40, generator=g, dtype=torch.float64) * 3
    bo = torch.randn(2, 3, 40, 16, generator=g, dtype=torch.float64)
    bl = torch.randn(2, 3, 40, generator=g, dtype=torch.float64) * 3
    no, nl = O.merge_closed_form(out, lse, bo, bl)
    np.savez_compressed(os.path.join(HERE, "merge_fold.npz"), out=out.numpy(), lse=lse.numpy(),
                        block_out=bo.numpy(), block_lse=bl.numpy(), new_out=no.numpy(), new_lse=nl.numpy())
    print("golden fixtures written to", HERE)


if __name__ == "__main__":
    main()

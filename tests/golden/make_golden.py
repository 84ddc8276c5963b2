"""Writes tests/golden/framed_pe_small.npz: inputs and float64 oracle outputs of one small problem.

The reference holds no golden vectors for this path and its kernels cannot be run here, so these
vectors come from this repository's own float64 oracle (oracle/torch_oracle.py), which
tests/test_oracle_pins.py pins against closed forms and brute force.  They freeze the oracle: a later
change to it that moves any number shows up as a test failure on the CPU, and the GPU kernels are
compared with the same frozen numbers.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import helpers as Hh                      # noqa: E402
from oracle import torch_oracle as TO     # noqa: E402

CUT = -3.5


def main():
    P = Hh.make_problem(num_crystals=5, atoms_lo=1, atoms_hi=5, seed=4242)
    a = P.a.clone().requires_grad_(True)
    Wk = P.W_k.clone().requires_grad_(True)
    Wax = [w.clone().requires_grad_(True) for w in P.W_ax]
    z, psi = TO.framed_pe(a, P.rpos, P.tvecs, P.batch, P.edges, Wk, Wax, P.frames, K=64, A=64, cos_abs=0,
                          c_dist=1.0, c_angle=1.0, rvlen=P.rvlen, cutoff_radius=CUT, windows="reference")
    ((z * P.gz).sum() + (psi * P.gpsi).sum()).backward()
    f1, f2, gap1, gap2 = TO.frame_axes_max(P.q, P.k, P.a, P.rpos, P.tvecs, P.batch, P.edges, rvlen=P.rvlen,
                                           cutoff_radius=CUT, return_gaps=True)
    out, prob = TO.softmax_attention(P.q, P.k, P.v, z.detach(), psi.detach(), P.batch, P.edges)
    arrays = dict(
        sizes=np.array(P.sizes), batch=P.batch.numpy(), edges=P.edges.numpy(), a=P.a.numpy(), rpos=P.rpos.numpy(),
        tvecs=P.tvecs.numpy(), rvlen=P.rvlen.numpy(), q=P.q.numpy(), k=P.k.numpy(), v=P.v.numpy(),
        W_k=P.W_k.numpy(), W_ax=np.stack([w.numpy() for w in P.W_ax]), frames=np.stack([f.numpy() for f in P.frames]),
        gz=P.gz.numpy(), gpsi=P.gpsi.numpy(),
        z=z.detach().numpy(), psi=psi.detach().numpy(), ga=a.grad.numpy(), gW_k=Wk.grad.numpy(),
        gW_ax=np.stack([w.grad.numpy() for w in Wax]), frame1=f1.numpy(), frame2max=f2.numpy(),
        gap1=gap1.numpy(), gap2=gap2.numpy(), attn_out=out.numpy(), attn_prob=prob.numpy())
    path = os.path.join(HERE, "framed_pe_small.npz")
    np.savez_compressed(path, **arrays)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()

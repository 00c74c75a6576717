"""Writes tests/golden/kfac_small.npz: small seeded inputs of every stage of the
per-layer K-FAC path together with what the NumPy oracle (oracle/kfac_oracle.py,
the restatement of the reference's --no_cuda arithmetic) returns for them.

The reference ships no vectors of its own and cannot be imported here (it needs
chainer and cupy), so these fixtures pin the oracle against itself over time and
give the GPU tests a fixed set of cases; the oracle's formulas are pinned by the
independent checks of tests/test_oracle_*.py.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from oracle import kfac_oracle as O   # noqa: E402


def build():
    r = np.random.default_rng(20240607)
    f32 = np.float32
    out = {}
    # linear layer, batch 12: A with bias column, G
    x = r.random((12, 37), dtype=f32)
    gy = (r.standard_normal((12, 9)) / 12).astype(f32)
    out.update(lin_x=x, lin_gy=gy, lin_A=O.linear_A(x, True), lin_G=O.linear_G(gy))
    # 3x3 convolution, pad 1 (bias) and a strided 1x1 convolution (no bias)
    cx = r.standard_normal((3, 5, 9, 8)).astype(f32)
    out.update(conv_x=cx, conv_A_k3s1p1=O.conv_A(cx, 3, 1, 1, True), conv_A_k1s2p0=O.conv_A(cx, 1, 2, 0, False),
               conv_A_k3s2p1=O.conv_A(cx, 3, 2, 1, True))
    cgy = (r.standard_normal((3, 6, 9, 8)) / 3).astype(f32)
    out.update(conv_gy=cgy, conv_G=O.conv_G(cgy))
    # batch normalisation, 4-D
    bx = r.standard_normal((6, 7, 5, 4)).astype(f32)
    bgy = (r.standard_normal((6, 7, 5, 4)) / 6).astype(f32)
    out.update(bn_x=bx, bn_gy=bgy, bn_grad=O.bn_grad_matrix(bx, bgy, 2e-5), bn_F=O.bn_F(bx, bgy, 2e-5))
    # damping + inverse of a connection block's factors
    A = O.conv_A(cx, 3, 1, 1, True).copy()
    G = O.conv_G(cgy).copy()
    (dA, dG), _ = O.connection_diagvals(A, G, 1e-2)
    out.update(damp_A_in=A.copy(), damp_G_in=G.copy(), damp_pi=np.float32(O.compute_pi(A, G)))
    Ad = A.copy(); Gd = G.copy()
    O.damp_inplace(Ad, dA); O.damp_inplace(Gd, dG)
    out.update(damp_A_out=Ad, damp_G_out=Gd, inv_A=O.inverse(Ad.copy()), inv_G=O.inverse(Gd.copy()))
    # preconditioning
    gW = r.standard_normal((6, 5, 3, 3)).astype(f32)
    gb = r.standard_normal(6).astype(f32)
    kW, kb = O.precondition_conn(out['inv_A'], out['inv_G'], gW, gb)
    out.update(pre_gW=gW, pre_gb=gb, pre_kW=kW, pre_kb=kb)
    Fd = O.bn_F(bx, bgy, 2e-5).copy()
    O.damp_inplace(Fd, O.bn_diagvals(7, 7, 1e-2, 16.0)[0])
    Finv = O.inverse(Fd.copy())
    gg = r.standard_normal(7).astype(f32); gbeta = r.standard_normal(7).astype(f32)
    kg, kbt, nan = O.precondition_bn(Finv, gg, gbeta)
    assert not nan
    out.update(bn_Finv=Finv, bn_gg=gg, bn_gbeta=gbeta, bn_kg=kg, bn_kbeta=kbt)
    # wire format: two triangular factors and a flat array, packed lower triangles
    arrays = [[(out['lin_A'], True), (gb, False), (out['conv_G'], True)]]
    buf = np.zeros(O.get_nelems(arrays), dtype=f32)
    O.pack(arrays, buf)
    out.update(pack_buf=buf)
    return {k: np.ascontiguousarray(v) for k, v in out.items()}


if __name__ == '__main__':
    np.savez_compressed(os.path.join(HERE, 'kfac_small.npz'), **build())
    print('wrote', os.path.join(HERE, 'kfac_small.npz'))

"""Pins the oracle's convolution / pooling / GEMM restatements against
independent statements: brute-force loops, torch CPU operators and adjoint
identities (no GPU needed)."""
import numpy as np
import pytest
import torch
import torch.nn.functional as TF

import oracle as orc


def brute_conv_fprop(I, F, pad, strd):
    C, D, H, W, N = I.shape
    _, T, R, S, K = F.shape
    M, P, Q = orc.conv_out_dims((D, H, W), (T, R, S), pad, strd)
    O = np.zeros((K, M, P, Q, N))
    for k in range(K):
        for m in range(M):
            for p in range(P):
                for q in range(Q):
                    for c in range(C):
                        for t in range(T):
                            for r in range(R):
                                for s in range(S):
                                    z = m * strd[0] - pad[0] + t
                                    y = p * strd[1] - pad[1] + r
                                    x = q * strd[2] - pad[2] + s
                                    if 0 <= z < D and 0 <= y < H and 0 <= x < W:
                                        O[k, m, p, q, :] += F[c, t, r, s, k] * I[c, z, y, x, :]
    return O


def test_conv_fprop_brute_force_tiny():
    rng = np.random.default_rng(0)
    I = rng.standard_normal((2, 3, 5, 4, 2))
    F = rng.standard_normal((2, 2, 3, 2, 3))
    pad, strd = (1, 1, 0), (1, 2, 1)
    got = orc.ref_conv_fprop(I, F, pad, strd)
    np.testing.assert_allclose(got, brute_conv_fprop(I, F, pad, strd), rtol=1e-5, atol=1e-6)


CONV_CASES = [
    # C, D,H,W, K, T,R,S, pad, stride, N
    (3, 1, 9, 9, 8, 1, 3, 3, (0, 1, 1), (1, 1, 1), 4),
    (4, 1, 11, 10, 8, 1, 5, 3, (0, 2, 1), (1, 2, 3), 2),
    (3, 1, 23, 23, 4, 1, 11, 11, (0, 2, 2), (1, 4, 4), 2),
    (2, 5, 6, 7, 4, 3, 3, 3, (1, 0, 1), (1, 1, 2), 2),
]


def _torch_conv(I, F, pad, strd):
    It = torch.from_numpy(np.transpose(I, (4, 0, 1, 2, 3)).copy()).requires_grad_(True)   # N C D H W
    Ft = torch.from_numpy(np.transpose(F, (4, 0, 1, 2, 3)).copy()).requires_grad_(True)   # K C T R S
    O = TF.conv3d(It, Ft, stride=strd, padding=pad)
    return It, Ft, O


@pytest.mark.parametrize("case", CONV_CASES)
def test_conv_against_torch_and_adjoint(case):
    C, D, H, W, K, T, R, S, pad, strd, N = case
    rng = np.random.default_rng(1)
    I = rng.standard_normal((C, D, H, W, N))
    F = rng.standard_normal((C, T, R, S, K))
    O = orc.ref_conv_fprop(I, F, pad, strd)
    It, Ft, Ot = _torch_conv(I, F, pad, strd)
    Ot_np = np.transpose(Ot.detach().numpy(), (1, 2, 3, 4, 0))
    # the reference rounds the output extent up; torch floors: compare the common part
    m, p, q = Ot_np.shape[1:4]
    np.testing.assert_allclose(O[:, :m, :p, :q, :], Ot_np, rtol=1e-4, atol=1e-5)
    if O.shape[1:4] != Ot_np.shape[1:4]:
        pytest.skip("ceil-mode extent: torch autograd not comparable")
    E = rng.standard_normal(O.shape)
    Ot.backward(torch.from_numpy(np.transpose(E, (4, 0, 1, 2, 3)).copy()))
    gI = np.transpose(It.grad.numpy(), (1, 2, 3, 4, 0))
    gF = np.transpose(Ft.grad.numpy(), (1, 2, 3, 4, 0))
    B = orc.ref_conv_bprop(F, E, I.shape, pad, strd)
    U = orc.ref_conv_update(I, E, F.shape, pad, strd)
    np.testing.assert_allclose(B, gI, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(U, gF, rtol=1e-4, atol=1e-4)
    # adjoint identity <fprop(I,F),E> == <I,bprop(F,E)> == <F,update(I,E)>
    a = np.vdot(O.astype(np.float64), E)
    np.testing.assert_allclose(np.vdot(I, B.astype(np.float64)), a, rtol=1e-5)
    np.testing.assert_allclose(np.vdot(F, U.astype(np.float64)), a, rtol=1e-5)


@pytest.mark.parametrize("case", CONV_CASES)
def test_conv_sampled_forms_match_full(case):
    C, D, H, W, K, T, R, S, pad, strd, N = case
    rng = np.random.default_rng(2)
    I = rng.standard_normal((C, D, H, W, N)).astype(np.float32)
    F = rng.standard_normal((C, T, R, S, K)).astype(np.float32)
    O = orc.ref_conv_fprop(I, F, pad, strd)
    E = rng.standard_normal(O.shape).astype(np.float32)
    M, P, Q = O.shape[1:4]
    pix = [(rng.integers(M), rng.integers(P), rng.integers(Q)) for _ in range(6)] + [(0, 0, 0), (M - 1, P - 1, Q - 1)]
    got = orc.ref_conv_fprop_pixels(I, F, pix, pad, strd)
    for i, (m, p, q) in enumerate(pix):
        np.testing.assert_allclose(got[i], O[:, m, p, q, :], rtol=1e-5, atol=1e-5)
    B = orc.ref_conv_bprop(F, E, I.shape, pad, strd)
    ipix = [(rng.integers(D), rng.integers(H), rng.integers(W)) for _ in range(6)] + [(0, 0, 0), (D - 1, H - 1, W - 1)]
    gotb = orc.ref_conv_bprop_pixels(F, E, I.shape, ipix, pad, strd)
    for i, (z, y, x) in enumerate(ipix):
        np.testing.assert_allclose(gotb[i], B[:, z, y, x, :], rtol=1e-5, atol=1e-5)
    U = orc.ref_conv_update(I, E, F.shape, pad, strd).reshape(-1, K)
    rows = rng.integers(0, U.shape[0], 5)
    gotu = orc.ref_conv_update_rows(I, E, F.shape, rows, pad, strd)
    np.testing.assert_allclose(gotu, U[rows], rtol=1e-4, atol=1e-4)


def brute_pool(I, op, JTRS, pad, strd):
    C, D, H, W, N = I.shape
    J, T, R, S = JTRS
    K, M, P, Q = orc.pool_out_dims((C, D, H, W), JTRS, pad, strd)
    O = np.zeros((K, M, P, Q, N))
    B_arg = {}
    for k in range(K):
        for m in range(M):
            for p in range(P):
                for q in range(Q):
                    for n in range(N):
                        best, arg, tot = -3.4028234663852886e38, None, 0.0
                        first = True
                        for j in range(J):
                            for t in range(T):
                                for r in range(R):
                                    for s in range(S):
                                        c = k * strd[0] - pad[0] + j
                                        z = m * strd[1] - pad[1] + t
                                        y = p * strd[2] - pad[2] + r
                                        x = q * strd[3] - pad[3] + s
                                        inb = 0 <= c < C and 0 <= z < D and 0 <= y < H and 0 <= x < W
                                        v = I[c, z, y, x, n] if inb else None
                                        if inb:
                                            tot += v
                                            if v > best:
                                                best, arg = v, (c, z, y, x)
                        O[k, m, p, q, n] = best if op == "max" else tot / (J * T * R * S)
                        B_arg[(k, m, p, q, n)] = arg
    return O, B_arg


POOL_CASES = [
    # C,D,H,W,N, JTRS, pad, stride
    (4, 1, 8, 8, 2, (1, 1, 2, 2), (0, 0, 0, 0), (1, 1, 2, 2)),
    (4, 1, 9, 9, 2, (1, 1, 3, 3), (0, 0, 0, 0), (1, 1, 2, 2)),
    (6, 1, 7, 7, 2, (2, 1, 3, 3), (0, 0, 1, 1), (2, 1, 2, 2)),
    (3, 4, 6, 5, 2, (1, 2, 3, 2), (0, 1, 1, 0), (1, 1, 2, 1)),
]


@pytest.mark.parametrize("case", POOL_CASES)
@pytest.mark.parametrize("op", ["max", "avg"])
def test_pool_brute_force(case, op):
    C, D, H, W, N, JTRS, pad, strd = case
    rng = np.random.default_rng(3)
    I = rng.standard_normal((C, D, H, W, N)).astype(np.float32)
    O = orc.ref_pool_fprop(I, op, JTRS, pad, strd)
    Ob, arg = brute_pool(I, op, JTRS, pad, strd)
    np.testing.assert_allclose(O, Ob, rtol=1e-6, atol=1e-6)
    E = rng.standard_normal(O.shape).astype(np.float32)
    B = orc.ref_pool_bprop(I, E, op, JTRS, pad, strd)
    if op == "max":
        Bb = np.zeros(I.shape)
        for (k, m, p, q, n), a in arg.items():
            if a is not None:
                Bb[a + (n,)] += E[k, m, p, q, n]
        np.testing.assert_allclose(B, Bb, rtol=1e-6, atol=1e-6)
    else:
        # adjoint identity <avg(I), E> == <I, avg_bprop(E)>
        np.testing.assert_allclose(np.vdot(O.astype(np.float64), E), np.vdot(I, B.astype(np.float64)), rtol=1e-5)
    wins = [(0, 0, 0, 0), tuple(d - 1 for d in O.shape[:4])]
    got = orc.ref_pool_fprop_pixels(I, op, JTRS, wins, pad, strd)
    for i, w in enumerate(wins):
        np.testing.assert_allclose(got[i], O[w], rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("case", POOL_CASES)
def test_l2_pool_closed_forms(case):
    """l2 pooling (benchmarks/pool_test.py:145-146) pinned without restating it: on inputs of
    constant magnitude c it is c * sqrt(number of window slots inside the tensor); it is positively
    homogeneous; and its square is the window SUM of I^2, i.e. J*T*R*S times the avg pooling of I^2."""
    C, D, H, W, N, JTRS, pad, strd = case
    rng = np.random.default_rng(8)
    sign = rng.choice([-1.0, 1.0], (C, D, H, W, N)).astype(np.float32)
    inside = orc.ref_pool_fprop(np.ones_like(sign), "avg", JTRS, pad, strd) * np.prod(JTRS)   # slots inside
    np.testing.assert_allclose(orc.ref_pool_fprop(0.75 * sign, "l2", JTRS, pad, strd), 0.75 * np.sqrt(inside), rtol=1e-6)
    I = rng.standard_normal((C, D, H, W, N)).astype(np.float32)
    O = orc.ref_pool_fprop(I, "l2", JTRS, pad, strd)
    np.testing.assert_allclose(orc.ref_pool_fprop(-3.0 * I, "l2", JTRS, pad, strd), 3.0 * O, rtol=1e-6)
    np.testing.assert_allclose(O.astype(np.float64) ** 2,
                               orc.ref_pool_fprop(I * I, "avg", JTRS, pad, strd).astype(np.float64) * np.prod(JTRS),
                               rtol=1e-5, atol=1e-6)
    # a 1x1x1x1 window is the absolute value
    np.testing.assert_allclose(orc.ref_pool_fprop(I, "l2", (1, 1, 1, 1)), np.abs(I), rtol=1e-6)


def test_pool_against_torch():
    rng = np.random.default_rng(4)
    I = rng.standard_normal((5, 1, 12, 12, 3)).astype(np.float32)
    It = torch.from_numpy(np.transpose(I[:, 0], (3, 0, 1, 2)).copy()).requires_grad_(True)  # N C H W
    Ot = TF.max_pool2d(It, 3, 2)
    O = orc.ref_pool_fprop(I, "max", (1, 1, 3, 3), (0, 0, 0, 0), (1, 1, 2, 2))
    np.testing.assert_array_equal(O[:, 0], np.transpose(Ot.detach().numpy(), (1, 2, 3, 0)))
    E = rng.standard_normal(O.shape).astype(np.float32)
    Ot.backward(torch.from_numpy(np.transpose(E[:, 0], (3, 0, 1, 2)).copy()))
    B = orc.ref_pool_bprop(I, E, "max", (1, 1, 3, 3), (0, 0, 0, 0), (1, 1, 2, 2))
    np.testing.assert_allclose(B[:, 0], np.transpose(It.grad.numpy(), (1, 2, 3, 0)), rtol=1e-5, atol=1e-6)
    Oa = orc.ref_pool_fprop(I, "avg", (1, 1, 3, 3), (0, 0, 1, 1), (1, 1, 2, 2))
    Ota = TF.avg_pool2d(It, 3, 2, padding=1, count_include_pad=True)
    np.testing.assert_allclose(Oa[:, 0], np.transpose(Ota.detach().numpy(), (1, 2, 3, 0)), rtol=1e-5, atol=1e-6)


def test_dot_known_answers_and_batched():
    # all-ones known answer: every element of C equals k (gemm_test2.py:40-41, test.cu:42-51)
    for size in (257, 128, 65, 17, 15):
        A = np.ones((size, size), np.float32)
        assert np.all(orc.ref_dot(A, A) == size)
    rng = np.random.default_rng(5)
    A = rng.standard_normal((4, 7, 5))
    B = rng.standard_normal((4, 5, 3))
    C = rng.standard_normal((4, 7, 3))
    got = orc.ref_batched_dot(A, B, C, alpha=0.5, beta=0.25, relu=True)
    exp = np.maximum(0.5 * np.einsum("bik,bkj->bij", A, B), 0) + 0.25 * C
    np.testing.assert_allclose(got, exp, rtol=1e-6)
    got2 = orc.ref_batched_dot(A, B, out_3d=False)
    np.testing.assert_allclose(got2, np.einsum("bik,bkj->ij", A, B), rtol=1e-6)
    got3 = orc.ref_batched_dot(A[0], B)
    np.testing.assert_allclose(got3, np.einsum("ik,bkj->bij", A[0], B), rtol=1e-6)


def test_ew_bn_closed_form_and_stack():
    rng = np.random.default_rng(6)
    A = rng.uniform(0, 1, (16, 64)).astype(np.float16)
    n = A.shape[1]
    c = 1.0 / n
    stack = [A, A, {"op": "sum", "axis": 1}, c, {"op": "mul"}, {"op": "sub"},
             A, A, {"op": "sum", "axis": 1}, c, {"op": "mul"}, {"op": "sub"}, {"op": "sqr"},
             {"op": "sum", "axis": 1}, c, {"op": "mul"}, 1e-3, {"op": "add"}, {"op": "sqrt"}, {"op": "div"}]
    got = orc.ref_ew(stack, A.shape)
    np.testing.assert_allclose(got, orc.ref_batchnorm_rows(A, 1e-3), rtol=2e-5, atol=2e-6)
    # mean 0 / variance 1-eps-ish per row
    assert np.allclose(got.mean(axis=1), 0, atol=1e-5)


def test_compensated_sum_tracks_fp64():
    rng = np.random.default_rng(7)
    s = np.zeros(256, np.float16)
    c = np.zeros(256, np.float16)
    tot = np.zeros(256, np.float64)
    plain = np.zeros(256, np.float16)
    for _ in range(400):
        a = rng.uniform(0, 0.01, 256).astype(np.float16)
        s, c = orc.ref_compensated_sum(s, c, a)
        plain = (plain.astype(np.float32) + a.astype(np.float32)).astype(np.float16)
        tot += a.astype(np.float64)
    err_k = np.abs(s.astype(np.float64) - tot).max()
    err_p = np.abs(plain.astype(np.float64) - tot).max()
    assert err_k <= 2 ** -10 * 4 and err_k < err_p / 4


def test_transpose_dimshuffle():
    F = np.arange(2 * 3 * 4 * 5 * 6).reshape(2, 3, 4, 5, 6)
    out = orc.ref_dimshuffle(F)
    assert out.shape == (6, 3, 4, 5, 2) and out[5, 2, 3, 4, 1] == F[1, 2, 3, 4, 5]
    assert orc.ref_transpose(F.reshape(6, -1))[7, 3] == F.reshape(6, -1)[3, 7]

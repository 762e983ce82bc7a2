"""Seeded synthetic problems and the acceptance metrics shared by the GPU parity tests."""
import numpy as np
import torch

MAX_REL_TOL = 1e-2     # max |out - ref| / max(|ref|, rms(ref))
NRMS_TOL = 1e-3        # ||out - ref||_2 / ||ref||_2


def make_problem(seed, M, N, K, nbits, GS, sym=False):
    """GPTQ-orientation inputs: activations fp16 ~N(0,1); weights int32 U{0..2^b-1} (K,N);
    scales fp16 ~U(0.001,0.02) (K/GS,N); zeros int32 U{0..2^b-1} (K/GS,N) or None."""
    g = torch.Generator().manual_seed(seed)
    A = torch.randn(M, K, generator=g).to(torch.float16)
    weight = torch.randint(0, 2 ** nbits, (K, N), dtype=torch.int32, generator=g)
    if GS == -1:
        return A, weight, None, None
    scale = (torch.rand(K // GS, N, generator=g) * 0.019 + 0.001).to(torch.float16)
    zero = None if sym else torch.randint(0, 2 ** nbits, (K // GS, N), dtype=torch.int32, generator=g)
    return A, weight, scale, zero


def reference_output(oracle, A, w, s, z, nbits, GS, rows=None):
    """Oracle forward from the PACKED tensors (numpy); ``rows`` restricts to some output columns."""
    A = A.cpu().numpy()
    w = w.cpu().numpy()
    if rows is not None:
        w = w[rows]
    if GS == -1:
        return oracle.gemv_plain_np(A, w, nbits)
    s = s.cpu().numpy()
    z = None if z is None else z.cpu().numpy()
    if rows is not None:
        s = s[rows]
        z = None if z is None else z[rows]
    out = np.empty((A.shape[0], w.shape[0]), dtype=np.float16)
    step = 4096
    for i in range(0, w.shape[0], step):
        out[:, i:i + step] = oracle.qlinear_np(A, w[i:i + step], s[i:i + step],
                                               None if z is None else z[i:i + step], nbits, GS)
    return out


def assert_close(oracle, out, ref, what=""):
    m = oracle.error_metrics(out, ref)
    assert np.all(np.isfinite(np.asarray(out, dtype=np.float32))), f"{what}: non-finite output"
    assert m["max_rel"] <= MAX_REL_TOL and m["nrms"] <= NRMS_TOL, f"{what}: {m}"
    return m

#!/usr/bin/env python3
"""Writes tests/golden/convert_fixtures.npz: seeded (weight, scale, zero) inputs and the packed (w, s, z) the
REFERENCE's own packer produces for them.

Runs in the build container only.  It loads the reference's ``qfactory/convert.py`` by file path (that file
imports nothing but torch; loading the package would pull in its nvcc JIT) and calls its ``convert_params`` on
CPU tensors.  Only data -- inputs and outputs -- is written; no reference source travels anywhere.  The tests
that consume the file (tests/test_golden.py) read the .npz and never touch the reference.

    python tests/golden/make_convert_fixtures.py [/root/reference]
"""
import importlib.util
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
# (nbits, K, N, GS): K a multiple of 32/nbits words, K/GS a whole number of zero-point bytes
CASES = [(b, K, N, GS)
         for b in (2, 4, 8)
         for (K, N) in ((32, 3), (64, 5), (256, 8))
         for GS in ({2: (8,), 4: (16,), 8: (16,)}[b] if K == 32 else (16, 32) if K == 64 else (32, 64))
         if (K // GS) % (8 // b) == 0]


def main():
    ref_root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    path = os.path.join(ref_root, "qfactory", "convert.py")
    spec = importlib.util.spec_from_file_location("reference_convert", path)
    ref = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(ref)

    out = {}
    names = []
    for idx, (b, K, N, GS) in enumerate(CASES):
        rng = np.random.default_rng(1000 + idx)
        weight = rng.integers(0, 2 ** b, size=(K, N), dtype=np.int32)
        scale = rng.uniform(0.001, 0.02, size=(K // GS, N)).astype(np.float16)
        zero = rng.integers(0, 2 ** b, size=(K // GS, N), dtype=np.int32)
        # the two ends of the range in every case: 0 and 2^b - 1 (the latter hits the packer's clamp)
        zero.flat[0], zero.flat[-1] = 0, 2 ** b - 1
        weight.flat[0], weight.flat[-1] = 2 ** b - 1, 0
        w, s, z = ref.convert_params({"K": K, "N": N, "NBITS": b, "GS": GS},
                                     (torch.from_numpy(weight), torch.from_numpy(scale), torch.from_numpy(zero)))
        w_plain = ref.convert_params({"K": K, "N": N, "NBITS": b}, (torch.from_numpy(weight),))
        w_sym, s_sym, z_sym = ref.convert_params({"K": K, "N": N, "NBITS": b, "GS": GS},
                                                 (torch.from_numpy(weight), torch.from_numpy(scale), None))
        assert z_sym is None and torch.equal(w_sym, w) and torch.equal(w_plain, w) and torch.equal(s_sym, s)
        name = f"b{b}_K{K}_N{N}_GS{GS}"
        names.append(name)
        out[name + "/weight"], out[name + "/scale"], out[name + "/zero"] = weight, scale, zero
        out[name + "/w"], out[name + "/s"], out[name + "/z"] = w.numpy(), s.numpy(), z.numpy()
        assert w.dtype == torch.int8 and z.dtype == torch.int8 and s.dtype == torch.float16
    out["names"] = np.array(names)
    target = os.path.join(HERE, "convert_fixtures.npz")
    np.savez_compressed(target, **out)
    print(f"wrote {target}: {len(names)} cases, {os.path.getsize(target)} bytes")


if __name__ == "__main__":
    main()

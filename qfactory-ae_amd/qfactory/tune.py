"""Tiling search with a persisted result.

The reference times every candidate of its search space at construction and can be pointed at a
JSON of earlier winners through ``$QFACTORY_CONFIG`` (qfactory/core/matmul.py:68-117; schema of
reproduce/*/best_config.json: ``"{nbits}-{m}-{n}-{k}-{group_size}" -> {attribute: value}``).  This
module is the writer of such a file for MI355X: run the on-device search once per shape, store the
winners, and later processes construct their layers without searching.

    python -m qfactory.tune --out best_config.json --shape 4 1 4096 4096 128 --shape 4 16 22016 4096 128
"""
import argparse
import json
import os

import torch

PERSISTED = ("regime", "parallel_strategy", "decode_strategy", "l2cache_a", "l2cache_b", "smem_quant", "tiling_configs")


def shape_key(nbits, m, n, k, group_size):
    return f"{nbits}-{m}-{n}-{k}-{group_size}"


def entry_of(qfunc):
    """The attributes of a specialisation that ``compile_profile`` restores from a config file."""
    return {name: getattr(qfunc, name) for name in PERSISTED if hasattr(qfunc, name)}


def tune_shape(nbits, m, n, k, group_size, sym=False, schedule=False):
    """Search one shape on the device; returns (key, entry)."""
    from .core import Matmul, QMatmul
    if group_size == -1:
        op = Matmul(n, k, nbits, torch.float16, torch.int8)
        op.compile_profile(enable_schedule=schedule, enable_lower=True)
        return shape_key(nbits, 1, n, k, -1), entry_of(op.best_qfunc)
    op = QMatmul(m, n, k, nbits, sym, torch.float16, torch.int8, group_size)
    op.compile_profile(enable_transform=True, enable_schedule=schedule, enable_lower=True)
    return shape_key(nbits, m, n, k, group_size), entry_of(op.best_qfunc)


def update_config(path, entries):
    """Merge ``entries`` into the JSON at ``path`` (atomic replace)."""
    config = {}
    if os.path.exists(path):
        with open(path) as f:
            config = json.load(f)
    config.update(entries)
    tmp = f"{path}.tmp.{os.getpid()}"
    with open(tmp, "w") as f:
        json.dump(config, f, indent=4, sort_keys=True)
    os.replace(tmp, path)
    return config


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--out", required=True)
    ap.add_argument("--shape", type=int, nargs=5, action="append", required=True,
                    metavar=("NBITS", "M", "N", "K", "GS"))
    ap.add_argument("--sym", action="store_true")
    ap.add_argument("--schedule", action="store_true", help="also try cached vs streaming weight loads")
    args = ap.parse_args()
    for nbits, m, n, k, gs in args.shape:
        key, entry = tune_shape(nbits, m, n, k, gs, sym=args.sym, schedule=args.schedule)
        update_config(args.out, {key: entry})
        print(key, json.dumps(entry), flush=True)


if __name__ == "__main__":
    main()

"""Writes tests/golden/space_filling_cluster.npz: inputs and outputs of the reference's balanced clustering.

The order `space_filling_cluster` (models/point_utils.py:61-208) produces depends on a float ranking key
(`mean_assignment * (dist_ratio.max() + 1) + dist_ratio`, point_utils.py:148-159) that no closed form pins, so
its vectors are taken from the function itself.  The module needs only `math` and `torch`; it is loaded by path,
on the CPU, in the container that holds the reference checkout.  The fixture holds data only: token positions in,
ranking / cluster centres / padding mask out.

    python tests/golden/make_cluster_vectors.py [/root/reference]
"""
import importlib.util
import os
import sys

import numpy as np
import torch


def load_point_utils(root):
    path = os.path.join(root, "models", "point_utils.py")
    spec = importlib.util.spec_from_file_location("_reference_point_utils", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def grid(h, w, b):
    ys, xs = torch.meshgrid(torch.arange(h), torch.arange(w), indexing="ij")
    return torch.stack([xs, ys], dim=2).reshape(1, -1, 2).expand(b, -1, -1).contiguous()


def subset(h, w, n, b, gen):
    full = grid(h, w, 1)[0]
    return torch.stack([full[torch.randperm(h * w, generator=gen)[:n]] for _ in range(b)])


def cases():
    gen = torch.Generator().manual_seed(20240607)
    yield "grid56", grid(56, 56, 2), 8, 56, 56
    yield "grid14", grid(14, 14, 2), 8, 14, 14
    yield "sub784", subset(56, 56, 784, 3, gen), 8, 56, 56
    yield "sub196", subset(56, 56, 196, 3, gen), 8, 56, 56
    yield "sub49", subset(56, 56, 49, 2, gen), 8, 56, 56
    yield "ref_script", subset(100, 100, 2499, 1, gen), 20, 100, 100
    yield "wide", subset(40, 72, 500, 2, gen), 8, 40, 72
    yield "grid96", grid(96, 96, 1), 8, 96, 96


def main():
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    ref = load_point_utils(root)
    out = {}
    names = []
    for name, pos, m, h, w in cases():
        new_pos, centres, member_idx, mask, ranking = ref.space_filling_cluster(pos.float(), m, h, w, no_reorder=False)
        centres_nr, member_nr, mask_nr = ref.space_filling_cluster(pos.float(), m, h, w, no_reorder=True)
        names.append(name)
        out[name + ".pos"] = pos.numpy().astype(np.int16)
        out[name + ".mhw"] = np.array([m, h, w], dtype=np.int32)
        out[name + ".ranking"] = ranking.squeeze(2).numpy().astype(np.int32)
        out[name + ".new_pos"] = new_pos.numpy().astype(np.float32)
        out[name + ".centres"] = centres.numpy().astype(np.float32)
        out[name + ".member_idx"] = member_idx.numpy().astype(np.int32)
        out[name + ".member_idx_no_reorder"] = member_nr.numpy().astype(np.int32)
        out[name + ".mask"] = (np.zeros((0,), np.uint8) if mask is None else mask.numpy().astype(np.uint8))
        assert torch.equal(centres, centres_nr)
    out["names"] = np.array(names)
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "space_filling_cluster.npz")
    np.savez_compressed(dst, **out)
    print("wrote", dst, os.path.getsize(dst), "bytes")


if __name__ == "__main__":
    main()

"""Writes tests/golden/layout_tables.npz from the reference's own layout functions.

Run once in the authoring container (the reference checkout is not available
anywhere else):  python tests/golden/make_golden.py

Only `triteia/python/ops/utils/sparsity.py` is loaded, by file path (it imports
nothing but torch and numpy); the package itself cannot be imported because it
pulls in a CUDA extension.  The functions captured here are the ones no
library routine or closed form pins independently:

  _get_perms_2_4                                (sparsity.py:35-61)
  _calculate_meta_reordering_scatter_offsets    (sparsity.py:134-161)
  sparse_semi_structured_from_dense_cutlass     (sparsity.py:167-290) on one
      small int32 matrix (codes + reorder end to end)
  mask_creator                                  (sparsity.py:99-118) on one
      tie-free input

The .npz holds inputs and outputs only.
"""
import importlib.util
import os

import numpy as np
import torch

REF = os.environ.get("TRITEIA_REFERENCE", "/root/reference")
SRC = os.path.join(REF, "triteia/python/ops/utils/sparsity.py")


def main():
    spec = importlib.util.spec_from_file_location("_ref_sparsity", SRC)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)

    out = {}
    perm, scale_perm, scale_perm_single = mod._get_perms_2_4()
    out["perm_2_4"] = perm.numpy().astype(np.int64)
    out["scale_perm_2_4"] = np.array(scale_perm, dtype=np.int64)
    out["scale_perm_single_2_4"] = np.array(scale_perm_single, dtype=np.int64)

    for (m, ncols) in [(64, 2), (128, 8), (256, 8), (256, 16), (512, 4)]:
        off = mod._calculate_meta_reordering_scatter_offsets(m, ncols, torch.int16, "cpu")
        out[f"meta_offsets_{m}_{ncols}"] = off.numpy().astype(np.int64)

    # one end-to-end encode: int32 matrix, 2 of 4 nonzero per group, values 1..15
    rng = np.random.default_rng(20240601)
    m, k = 64, 128
    dense = np.zeros((m, k // 4, 4), dtype=np.int32)
    for r in range(m):
        for g in range(k // 4):
            pos = rng.choice(4, size=2, replace=False)
            dense[r, g, pos] = rng.integers(1, 16, size=2)
    dense = dense.reshape(m, k)
    sparse, meta = mod.sparse_semi_structured_from_dense_cutlass(torch.from_numpy(dense))
    out["encode_in"] = dense
    out["encode_sparse"] = sparse.numpy().astype(np.int32)
    out["encode_meta"] = meta.numpy().astype(np.int16)
    back = mod.sparse_semi_structured_to_dense_cutlass(sparse, meta)
    out["encode_roundtrip_ok"] = np.array(bool((back == torch.from_numpy(dense)).all()))

    # encode with kept zeros (the nibble-0 hazard): some kept values are 0
    dense0 = dense.copy().reshape(m, k // 4, 4)
    kill = rng.random((m, k // 4)) < 0.2
    for r in range(m):
        for g in range(k // 4):
            if kill[r, g]:
                nzp = np.nonzero(dense0[r, g])[0]
                dense0[r, g, nzp[rng.integers(0, 2)]] = 0
    dense0 = dense0.reshape(m, k)
    sparse0, meta0 = mod.sparse_semi_structured_from_dense_cutlass(torch.from_numpy(dense0))
    out["encode0_in"] = dense0
    out["encode0_sparse"] = sparse0.numpy().astype(np.int32)
    out["encode0_meta"] = meta0.numpy().astype(np.int16)

    # mask_creator on a tie-free input
    x = rng.permutation(64 * 32).astype(np.float32).reshape(64, 32) + 1.0
    x *= rng.choice([-1.0, 1.0], size=x.shape)
    mask = mod.mask_creator(torch.from_numpy(x), n=2, m=4)
    out["mask_in"] = x
    out["mask_out"] = mask.numpy().astype(np.uint8)

    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "layout_tables.npz")
    np.savez_compressed(dst, **out)
    print("wrote", dst, {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()

"""The product's torch codec / generators against the oracle (CPU, bit-exact)."""
import numpy as np
import pytest
import torch

from oracle import triteia_oracle as orc
from triteia_amd.python.ops.utils import generator as gen
from triteia_amd.python.ops.utils import sparsity as sp


@pytest.mark.parametrize("k,m", [(128, 256), (256, 512), (512, 256), (192, 128)])
def test_pack_matches_oracle(k, m):
    g = torch.Generator().manual_seed(k + m)
    qw, s, meta, (q, lo, hi) = gen.gen_explicit_sparse_quant4(m, k, device="cpu", generator=g)
    if k % 128 == 0 and m % 256 == 0:
        qo, mo, so = orc.pack_explicit(q.numpy(), lo.numpy(), hi.numpy(), s.numpy())
        assert np.array_equal(qw.numpy(), qo)
        assert np.array_equal(meta.numpy(), mo)
        assert np.array_equal(s.numpy(), so)
        assert np.array_equal(sp.unpack_2_4(qw, meta, s).numpy(), orc.unpack(qo, mo, so))
        assert np.array_equal(sp.unpack_2_4(qw, meta).numpy().astype(np.int32), orc.unpack_int(qo, mo))
    assert torch.equal(sp.unpack_nibbles(qw), (q.t() + 8).to(torch.uint8))
    lo2, hi2 = sp.unpack_meta(meta)
    assert torch.equal(lo2, lo) and torch.equal(hi2, hi)


def test_mask_creator_matches_oracle_and_golden():
    import os
    G = np.load(os.path.join(os.path.dirname(__file__), "golden", "layout_tables.npz"))
    mask = sp.mask_creator(torch.from_numpy(G["mask_in"]))
    assert np.array_equal(mask.numpy().astype(np.uint8), G["mask_out"])
    with pytest.raises(ValueError):
        sp.mask_creator(torch.zeros(3, 3))


def test_reference_style_generator_roundtrip():
    g = torch.Generator().manual_seed(5)
    unc, q, s, meta = gen.gen_sparse_quant4_NT(256, 128, device="cpu", generator=g)
    assert unc.shape == (128, 256) and q.shape == (4, 512) and meta.shape == (256, 8) and s.shape == (1, 256)
    assert np.array_equal(orc.unpack(q.numpy(), meta.numpy(), s.numpy()), unc.numpy())
    # 2:4 structure
    nz = (unc.t().reshape(256, 32, 4) != 0).sum(-1)
    assert int(nz.max()) <= 2
    uncs, qs, ss, metas = gen.gen_batched_sparse_quant4_NT(3, 256, 128, device="cpu", generator=g)
    assert uncs.shape == (3, 128, 256) and qs.shape == (3, 4, 512) and ss.shape == (3, 1, 256)


def test_module_pack_equals_oracle_reference_packer():
    from triteia_amd.python.nn.linear import sparse_low_precision_linear
    g = torch.Generator().manual_seed(9)
    k, m = 128, 256
    w = torch.randn((k, m), generator=g).half()
    s = (w.abs().max(0, keepdim=True)[0] * (2 / 15)).half()
    mask = sp.mask_creator(w.t().contiguous())
    w24 = (mask.t() * w).half()
    layer = sparse_low_precision_linear(k, m)
    layer.pack(w24, s, True)
    q = torch.clamp(torch.round(w24 / s).int() + 8, 0, 15)
    if not bool(((q == 0) & mask.t().bool()).any()):
        qo, mo, so = orc.pack_reference(w24.numpy(), s.numpy(), mask=mask.bool().numpy())
        assert np.array_equal(layer.qweight.numpy(), qo)
        assert np.array_equal(layer.meta.numpy(), mo)
    W = orc.unpack(layer.qweight.numpy(), layer.meta.numpy(), layer.scale.numpy())
    expect = ((q - 8).half() * s * mask.t()).half()
    assert np.array_equal(W, expect.numpy())
    layer.pack(w24, s, True)   # packing twice is allowed


def test_pack_writes_where_the_reference_writes():
    """The reference's callers assign `B`, `s` and `meta` on the module and read the packed tensors back from
    them (generator.py:60-68); `pack` takes `trans` with the reference's default, and that default -- the
    dense-Marlin permutation, which nothing on this path reads -- raises instead of packing something else."""
    import inspect
    from triteia_amd.python.nn.linear import sparse_low_precision_linear
    g = torch.Generator().manual_seed(19)
    k, m = 128, 256
    w = torch.randn((k, m), generator=g).half()
    s = (w.abs().max(0, keepdim=True)[0] * (2 / 15)).half()
    mask = sp.mask_creator(w.t().contiguous())
    w24 = (mask.t() * w).half()
    assert inspect.signature(sparse_low_precision_linear.pack).parameters["trans"].default is False
    layer = sparse_low_precision_linear(k, m, groupsize=-1)
    layer.B = torch.empty((k // 2 // 16, m * 16 // 8), dtype=torch.int)
    layer.meta = torch.empty((m, k // 16), dtype=torch.int16)
    layer.s = torch.empty((1, m), dtype=torch.half)
    with pytest.raises(NotImplementedError, match="trans=True"):
        layer.pack(w24, s)
    layer.pack(w24, s, True)
    plain = sparse_low_precision_linear(k, m)
    plain.pack(w24, s, True)
    assert torch.equal(layer.B, plain.qweight) and torch.equal(layer.s, plain.scale) and torch.equal(layer.meta, plain.meta)
    assert torch.equal(layer.qweight, plain.qweight) and torch.equal(layer.scale, plain.scale)
    # fp16_to_sparse: the reference's five values; meta_raw is the metadata before the kernel's re-layout
    out = gen.fp16_to_sparse(w24, s, device="cpu")
    assert len(out) == 5
    _, q5, s5, meta5, raw5 = out
    assert torch.equal(q5, plain.qweight) and torch.equal(meta5, plain.meta) and torch.equal(raw5, plain.meta_raw)
    assert np.array_equal(orc.reorder_meta(raw5.numpy().view(np.uint16)).view(np.int16), meta5.numpy())
    assert np.array_equal(orc.unreorder_meta(meta5.numpy().view(np.uint16)).view(np.int16), raw5.numpy())


def test_model_distribution():
    for dist in ("uniform", "zipf:1.5", "rank-zipf:1.5"):
        idx = gen.generate_model_distribution(dist, 1000, 8, device="cpu", seed=3)
        assert idx.dtype == torch.int32 and idx.shape == (1000,)
        assert int(idx.min()) >= -1 and int(idx.max()) < 8
        again = gen.generate_model_distribution(dist, 1000, 8, device="cpu", seed=3)
        assert torch.equal(idx, again)
    z = gen.generate_model_distribution("rank-zipf:1.5", 4000, 8, device="cpu", seed=1)
    counts = torch.bincount(z.long(), minlength=8)
    assert counts[0] > counts[3] > counts[7]
    r = gen.generate_model_distribution("zipf:1.5", 4000, 8, device="cpu", seed=1)
    counts = torch.bincount((r + 1).long(), minlength=9)
    assert counts[8] > counts[1]     # the reference's law grows with the index


def test_tp_shards_are_packed_independently():
    g = torch.Generator().manual_seed(2)
    k, m = 256, 512
    w = torch.randn((k, m), generator=g).half()
    s = (w.abs().max(0, keepdim=True)[0] * (2 / 15)).half()
    mask = sp.mask_creator(w.t().contiguous())
    w24 = (mask.t() * w).half()
    qs, ss, ms = gen.torch_weight_to_sparse_marlin(w24, s, tp_size=2, chunk_by="column", device="cpu")
    full = orc.unpack(*(t.numpy() for t in gen.fp16_to_sparse(w24, s, device="cpu")[1:2]
                        + gen.fp16_to_sparse(w24, s, device="cpu")[3:4] + gen.fp16_to_sparse(w24, s, device="cpu")[2:3]))
    parts = [orc.unpack(q.numpy(), me.numpy(), sc.numpy()) for q, sc, me in zip(qs, ss, ms)]
    assert np.array_equal(np.concatenate(parts, axis=1), full)
    qs, ss, ms = gen.torch_weight_to_sparse_marlin(w24, s, tp_size=2, chunk_by="row", device="cpu")
    parts = [orc.unpack(q.numpy(), me.numpy(), sc.numpy()) for q, sc, me in zip(qs, ss, ms)]
    assert np.array_equal(np.concatenate(parts, axis=0), full)


def test_group_scales_codec_matches_the_oracle():
    from triteia_amd.python.ops.utils.sparsity import pack_group_scales, unpack_2_4, unpack_group_scales
    rng = np.random.default_rng(5)
    k, m = 256, 128
    s = (np.abs(rng.standard_normal((k // 128, m))) * 0.01 + 0.005).astype(np.float16)
    stored = pack_group_scales(torch.from_numpy(s))
    assert np.array_equal(stored.numpy(), orc.store_group_scales(s))
    assert np.array_equal(unpack_group_scales(stored).numpy(), s)
    w = (rng.standard_normal((k, m)) * 0.05).astype(np.float16)
    qw, meta, st = orc.pack_reference_grouped(w, s)
    W = unpack_2_4(torch.from_numpy(qw), torch.from_numpy(meta), torch.from_numpy(st))
    assert np.array_equal(W.numpy(), orc.unpack(qw, meta, st))

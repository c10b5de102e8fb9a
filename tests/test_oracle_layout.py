"""Pins the oracle's layout functions (CPU only).

Golden tables come from the reference's own functions (tests/golden/); the
2:4 code table is additionally pinned by the installed torch library.
"""
import os

import numpy as np
import pytest
import torch

from oracle import triteia_oracle as orc

G = np.load(os.path.join(os.path.dirname(__file__), "golden", "layout_tables.npz"))


def test_perm_matches_reference_table():
    perm = orc.perm_2_4()
    assert np.array_equal(perm, G["perm_2_4"])
    assert np.array_equal(np.sort(perm), np.arange(1024))
    assert np.array_equal(orc.perm_2_4_closed_form(), G["perm_2_4"])


def test_scale_perm_single_is_identity():
    # per-channel scales are stored un-permuted (sparsity.py:58-60)
    assert np.array_equal(G["scale_perm_single_2_4"], np.arange(64))


def test_group_scale_order_matches_reference_table():
    # scales per group of K are stored with every run of 8 columns in the order 0 4 1 5 2 6 3 7 (sparsity.py:54-57)
    assert np.array_equal(orc.scale_perm_2_4(), G["scale_perm_2_4"])
    assert np.array_equal(np.sort(orc.scale_perm_2_4()), np.arange(64))
    s = np.arange(3 * 128, dtype=np.float16).reshape(3, 128)
    stored = orc.store_group_scales(s)
    # column c of a run of 8 sits at position 0 2 4 6 1 3 5 7 [c] of that run
    for g in range(3):
        for col in range(128):
            assert stored[g, col // 8 * 8 + (0, 2, 4, 6, 1, 3, 5, 7)[col % 8]] == s[g, col]
    assert np.array_equal(orc.load_group_scales(stored), s)


def test_grouped_scales_against_a_plain_loop_and_the_per_column_form():
    rng = np.random.default_rng(77)
    k, m, T = 256, 256, 3
    w = (rng.standard_normal((k, m)) * 0.05).astype(np.float16)
    mask = orc.mask_2_4(np.ascontiguousarray(np.abs(w.T.astype(np.float32)) + rng.random((m, k)).astype(np.float32) * 1e-3))
    # (scales large enough that no kept weight reaches -8: the reference's packer takes nibble 0 for a pruned entry)
    s = (np.abs(rng.standard_normal((k // 128, m))) * 0.01 + 0.035).astype(np.float16)
    qw, meta, stored = orc.pack_reference_grouped(w, s, mask)
    assert stored.shape == (k // 128, m) and stored.dtype == np.float16
    W = orc.unpack(qw, meta, stored)
    q = orc.unpack_int(qw, meta)
    # every weight: its integer times the scale of (its group of 128 rows, its column), rounded to fp16; the integer is
    # the weight divided by that scale, rounded, clamped to int4, zero where pruned
    for kk in range(0, k, 5):
        for c in range(0, m, 3):
            sc = s[kk // 128, c]
            assert W[kk, c] == np.float16(np.float16(q[kk, c]) * sc)
            want = int(np.clip(np.rint(np.float32(np.float16(w[kk, c] / sc))), -8, 7)) if mask[c, kk] else 0
            assert q[kk, c] == want, (kk, c)
    x = rng.standard_normal((T, k)).astype(np.float16)
    y = orc.matmul_4bit_2_4(qw, x, meta, stored)
    for t in range(T):
        for c in range(0, m, 7):
            acc = sum(float(x[t, kk]) * float(W[kk, c]) for kk in range(k))
            assert abs(acc - y[t, c]) < 1e-9
    # all groups alike: the per-column result
    s1 = s[:1]
    qw1, meta1, stored1 = orc.pack_reference_grouped(w, np.repeat(s1, k // 128, axis=0), mask)
    qwc, metac, sc1 = orc.pack_reference(w, s1, mask)
    assert np.array_equal(qw1, qwc) and np.array_equal(meta1, metac)
    assert np.array_equal(orc.matmul_4bit_2_4(qw1, x, meta1, stored1), orc.matmul_4bit_2_4(qwc, x, metac, sc1))


@pytest.mark.parametrize("m,ncols", [(64, 2), (128, 8), (256, 8), (256, 16), (512, 4)])
def test_meta_offsets_match_reference_table(m, ncols):
    off = orc.meta_scatter_offsets(m, ncols)
    assert np.array_equal(off, G[f"meta_offsets_{m}_{ncols}"])
    assert np.array_equal(np.sort(off), np.arange(m * ncols))
    closed = np.array([orc.meta_offset_closed_form(r, c, m) for r in range(m) for c in range(ncols)])
    assert np.array_equal(closed, G[f"meta_offsets_{m}_{ncols}"])


def test_meta_block_is_contiguous_per_32k():
    # all metadata of one 32-dense-k block occupies one contiguous 2m-int16 run
    m, ncols = 256, 16
    off = G["meta_offsets_256_16"].reshape(m, ncols)
    for c in range(ncols):
        blk = off[:, c] // (2 * m)
        assert np.all(blk == c // 2)


def test_encode_matches_reference_vectors():
    for tag in ("encode", "encode0"):
        dense = G[f"{tag}_in"]
        sparse, meta16 = orc.encode_2_4_nonzero(dense)
        assert np.array_equal(sparse, G[f"{tag}_sparse"])
        assert np.array_equal(orc.reorder_meta(meta16).view(np.int16), G[f"{tag}_meta"])
    assert bool(G["encode_roundtrip_ok"])


def test_encode_codes_match_torch_library():
    # independent pin: torch's own CUTLASS-format encoder uses the same code table
    from torch.sparse import _semi_structured_conversions as lib

    rng = np.random.default_rng(7)
    m, k = 64, 256
    dense = np.zeros((m, k // 4, 4), dtype=np.float32)
    lo = np.empty((m, k // 4), dtype=np.int64)
    hi = np.empty((m, k // 4), dtype=np.int64)
    for r in range(m):
        for g in range(k // 4):
            a, b = sorted(rng.choice(4, size=2, replace=False))
            lo[r, g], hi[r, g] = a, b
            dense[r, g, [a, b]] = rng.integers(1, 16, size=2)
    dense = dense.reshape(m, k)
    sp_t, meta_t = lib.sparse_semi_structured_from_dense_cutlass(torch.from_numpy(dense).half())
    off_t = lib._calculate_meta_reordering_scatter_offsets(m, k // 16, torch.int16, "cpu")
    meta_logical_t = meta_t.reshape(-1)[off_t].reshape(m, k // 16).numpy().view(np.uint16)
    sparse, meta16 = orc.encode_2_4_nonzero(dense.astype(np.int32))
    assert np.array_equal(meta16, meta_logical_t)
    assert np.array_equal(sparse, sp_t.float().numpy().astype(np.int32))
    # explicit positions give the same codes when no kept value is zero
    _, meta16_e = orc.encode_2_4_explicit(sparse, lo, hi)
    assert np.array_equal(meta16_e, meta16)


def test_six_legal_patterns_code_table():
    # sparsity.py:212-218
    table = {(0, 1): 0b0100, (0, 2): 0b1000, (1, 2): 0b1001, (0, 3): 0b1100, (1, 3): 0b1101, (2, 3): 0b1110}
    for (a, b), code in table.items():
        d = np.zeros((1, 16), dtype=np.int32)
        for g in range(4):
            d[0, 4 * g + a] = 3
            d[0, 4 * g + b] = 5
        _, meta16 = orc.encode_2_4_nonzero(d)
        assert int(meta16[0, 0]) == code * 0x1111
        assert (a | (b << 2)) == code


def test_mask_matches_reference_vector():
    assert np.array_equal(orc.mask_2_4(G["mask_in"]).astype(np.uint8), G["mask_out"])


def _random_problem(rng, k, m, avoid_minus8=False):
    lo = np.empty((m, k // 4), dtype=np.int64)
    hi = np.empty((m, k // 4), dtype=np.int64)
    pairs = np.array([(0, 1), (0, 2), (0, 3), (1, 2), (1, 3), (2, 3)])
    sel = rng.integers(0, 6, size=(m, k // 4))
    lo[:], hi[:] = pairs[sel, 0], pairs[sel, 1]
    q = rng.integers(-7 if avoid_minus8 else -8, 8, size=(m, k // 2))
    s = rng.uniform(0.005, 0.02, size=m).astype(np.float16)
    return q, lo, hi, s


def _dense_from(q, lo, hi):
    m, k2 = q.shape
    k = 2 * k2
    d = np.zeros((m, k // 4, 4), dtype=np.int32)
    qq = q.reshape(m, k // 4, 2)
    np.put_along_axis(d, lo[..., None], qq[..., 0:1], axis=-1)
    np.put_along_axis(d, hi[..., None], qq[..., 1:2], axis=-1)
    return d.reshape(m, k).T  # [k, m]


@pytest.mark.parametrize("k,m", [(128, 256), (256, 512), (512, 256)])
def test_pack_unpack_roundtrip_exact(k, m):
    rng = np.random.default_rng(k * 7 + m)
    q, lo, hi, s = _random_problem(rng, k, m)
    qw, meta, sc = orc.pack_explicit(q, lo, hi, s)
    assert qw.shape == (k // 32, 2 * m) and qw.dtype == np.int32
    assert meta.shape == (m, k // 16) and meta.dtype == np.int16
    S, lo2, hi2 = orc.unpack_codes(qw, meta)
    assert np.array_equal(S.T.astype(np.int32) - 8, q)
    assert np.array_equal(lo2, lo) and np.array_equal(hi2, hi)
    assert np.array_equal(orc.unpack_int(qw, meta), _dense_from(q, lo, hi))


def test_pack_brute_force_minimum_size():
    # every nibble located through the closed form (lane, word, nibble), not the table pipeline
    k, m = 128, 256
    rng = np.random.default_rng(3)
    q, lo, hi, s = _random_problem(rng, k, m)
    qw, meta, _ = orc.pack_explicit(q, lo, hi, s)
    qu = qw.view(np.uint32)
    inter = [0, 2, 4, 6, 1, 3, 5, 7]
    for tr in range(k // 32):
        for chunk in range(m // 64):
            for i in range(32):
                for w in range(4):
                    word = int(qu[tr, 128 * chunk + 4 * i + w])
                    for n in range(8):
                        p = inter[n]
                        block, rsel = p // 4, p % 4
                        j = 16 * tr + 2 * (i % 4) + (rsel % 2) + 8 * (rsel // 2)
                        c = 64 * chunk + 8 * (i // 4) + 4 * block + w
                        assert ((word >> (4 * n)) & 15) == q[c, j] + 8
    mu = meta.view(np.uint16).ravel()
    for r in range(m):
        for c16 in range(k // 16):
            code16 = int(mu[orc.meta_offset_closed_form(r, c16, m)])
            for g in range(4):
                code = (code16 >> (4 * g)) & 15
                assert code & 3 == lo[r, 4 * c16 + g] and code >> 2 == hi[r, 4 * c16 + g]


def test_pack_reference_equals_explicit_without_nibble_zero():
    k, m = 128, 256
    rng = np.random.default_rng(11)
    q, lo, hi, s = _random_problem(rng, k, m, avoid_minus8=True)
    # make every kept value nonzero after the +8 shift (q != -8) -- then `!= 0`
    # detection in the reference packer sees exactly the kept positions
    dense_q = _dense_from(q, lo, hi)                     # [k, m]
    s16 = s.reshape(1, m)
    W = (dense_q.astype(np.float16) * s16).astype(np.float16)
    mask = np.zeros((m, k // 4, 4), dtype=bool)
    np.put_along_axis(mask, lo[..., None], True, axis=-1)
    np.put_along_axis(mask, hi[..., None], True, axis=-1)
    qw_r, meta_r, _ = orc.pack_reference(W, s16, mask=mask.reshape(m, k))
    qw_e, meta_e, _ = orc.pack_explicit(q, lo, hi, s)
    assert np.array_equal(qw_r, qw_e)
    assert np.array_equal(meta_r, meta_e)


def test_reference_packer_nibble_zero_hazard_is_real():
    # a kept -8 (nibble 0) is invisible to `!= 0` detection: the packed tensors then
    # decode to something other than the dense input; the explicit packer does not
    k, m = 128, 256
    rng = np.random.default_rng(12)
    q, lo, hi, s = _random_problem(rng, k, m)
    assert (q == -8).any()
    dense_q = _dense_from(q, lo, hi)
    qw_e, meta_e, _ = orc.pack_explicit(q, lo, hi, s)
    assert np.array_equal(orc.unpack_int(qw_e, meta_e), dense_q)


def test_single_nonzero_closed_form():
    k, m = 128, 256
    rng = np.random.default_rng(5)
    x = rng.standard_normal((3, k)).astype(np.float16)
    for (kk, c, val) in [(0, 0, 7), (77, 130, -8), (127, 255, 3), (34, 65, -1)]:
        lo = np.zeros((m, k // 4), dtype=np.int64)
        hi = np.ones((m, k // 4), dtype=np.int64)
        q = np.zeros((m, k // 2), dtype=np.int64)
        g, pos = kk // 4, kk % 4
        if pos == 0:
            lo[c, g], hi[c, g], slot = 0, 1, 0
        else:
            lo[c, g], hi[c, g], slot = 0, pos, 1
        q[c, 2 * g + slot] = val
        s = rng.uniform(0.005, 0.02, size=m).astype(np.float16)
        qw, meta, sc = orc.pack_explicit(q, lo, hi, s)
        y = orc.matmul_4bit_2_4(qw, x, meta, sc)
        expect = np.zeros((3, m))
        wv = np.float64(np.float16(np.float16(val) * s[c]))
        expect[:, c] = x[:, kk].astype(np.float64) * wv
        assert np.allclose(y, expect, rtol=0, atol=1e-12)


def test_all_ones_gives_column_sums():
    k, m = 128, 256
    rng = np.random.default_rng(6)
    q, lo, hi, _ = _random_problem(rng, k, m)
    q[:] = 1
    s = np.full(m, 0.0078125, dtype=np.float16)  # 2^-7: products exact
    qw, meta, sc = orc.pack_explicit(q, lo, hi, s)
    x = np.ones((2, k), dtype=np.float16)
    y = orc.matmul_4bit_2_4(qw, x, meta, sc)
    assert np.allclose(y, (k // 2) * 0.0078125)


def test_ops_against_python_loops():
    k, m, N, T = 128, 256, 3, 7
    rng = np.random.default_rng(9)
    packs = [orc.pack_explicit(*_random_problem(rng, k, m)) for _ in range(N)]
    qws = np.stack([p[0] for p in packs])
    metas = np.stack([p[1] for p in packs])
    ss = np.stack([p[2] for p in packs])
    x = rng.standard_normal((T, k)).astype(np.float16)
    idx = np.array([2, -1, 0, 0, 1, -1, 2], dtype=np.int32)
    y = orc.sbmm_4bit_2_4(qws, x, metas, ss, idx)
    dense = [orc.unpack(qws[d], metas[d], ss[d]) for d in range(N)]
    for t in range(T):
        if idx[t] < 0:
            assert np.all(y[t] == 0)
            continue
        W = dense[idx[t]]
        for c in range(0, m, 17):
            acc = 0.0
            for kk in range(k):
                acc += float(x[t, kk]) * float(W[kk, c])
            assert abs(acc - y[t, c]) < 1e-9
    # dense-weight form agrees
    y2 = orc.sbmm_dense(np.stack(dense), x, idx)
    assert np.allclose(y, y2, atol=1e-12)
    # bmm = one matrix per batch entry
    xb = rng.standard_normal((N, 2, k)).astype(np.float16)
    yb = orc.bmm_4bit_2_4(qws, xb, metas, ss)
    for b in range(N):
        assert np.allclose(yb[b], xb[b].astype(np.float64) @ dense[b].astype(np.float64))
    # lora + ldmm routing
    M, r = 2, 8
    A = rng.standard_normal((M, k, r)).astype(np.float16)
    B = rng.standard_normal((M, r, m)).astype(np.float16)
    lidx = np.array([0, 1, -1, 1, 0, -1, 0])
    yl = orc.lora(A, B, x, lidx)
    for t in range(T):
        if lidx[t] < 0:
            assert np.all(yl[t] == 0)
        else:
            v = np.array([sum(float(x[t, kk]) * float(A[lidx[t], kk, j]) for kk in range(k)) for j in range(r)])
            v = v.astype(np.float16).astype(np.float64)
            assert np.allclose(yl[t], v @ B[lidx[t]].astype(np.float64))
    mixed = np.array([0, 1, -1, 2, 3, 4, 1])  # <2 lora, >=2 delta (minus 2)
    ym = orc.ldmm(mixed, x, A, B, qws, metas, ss)
    for t in range(T):
        i = mixed[t]
        if i < 0:
            assert np.all(ym[t] == 0)
        elif i < M:
            assert np.allclose(ym[t], orc.lora(A, B, x[t:t + 1], np.array([i]))[0])
        else:
            assert np.allclose(ym[t], x[t].astype(np.float64) @ dense[i - M].astype(np.float64))


def test_round_bf16_against_the_torch_conversion():
    """The oracle's bfloat16 rounding (for the LoRA ops' bf16 instantiation) against torch's own conversion,
    ties included (0x3F808000 lies halfway between two bf16 values and goes to the even one)."""
    import torch
    rng = np.random.default_rng(5)
    a = np.concatenate([rng.standard_normal(20000) * 7, rng.standard_normal(2000) * 1e-3,
                        np.array([0x3F808000, 0x3F818000, 0x3F807FFF, 0x3F808001, 0xBF808000], dtype=np.uint32).view(np.float32)])
    want = torch.from_numpy(a.astype(np.float32)).to(torch.bfloat16).double().numpy()
    assert np.array_equal(orc.round_bf16(a), want)
    # and the lora restatement with that rounding against a plain loop
    A = orc.round_bf16(rng.standard_normal((2, 16, 8))).astype(np.float32)
    B = orc.round_bf16(rng.standard_normal((2, 8, 24))).astype(np.float32)
    x = orc.round_bf16(rng.standard_normal((5, 16))).astype(np.float32)
    idx = np.array([1, -1, 0, 1, 0])
    got = orc.lora(A, B, x, idx, intermediate="bf16")
    for t in range(5):
        if idx[t] < 0:
            assert not got[t].any()
            continue
        v = [float(torch.tensor(sum(float(x[t, i]) * float(A[idx[t], i, j]) for i in range(16)), dtype=torch.float32).to(torch.bfloat16))
             for j in range(8)]
        want_row = [sum(v[j] * float(B[idx[t], j, c]) for j in range(8)) for c in range(24)]
        assert np.allclose(got[t], want_row, rtol=1e-12, atol=1e-12)

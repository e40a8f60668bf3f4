"""Pins the CPU oracle (oracle/kv_oracle.py + oracle/kv_oracle.c) before it is trusted.

The reference holds no tests, fixtures or golden vectors for this path, so the
oracle is pinned by (1) three independent statements of each op agreeing
(reference torch expression / C loops / pure-Python element loops), (2) the
committed fixtures of tests/golden/, (3) what the mathematics fixes: round
trips, canary invariants, the identity slot mapping, and (4) for the one
floating-point rule, torch's own ``.to(torch.float8_e4m3fn)`` cast — the
library routine named as the contract — exhaustively over every 16-bit input.
"""
import hashlib
import json
import os

import numpy as np
import pytest
import torch

from oracle import kv_oracle as orc


def bits16(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def from_bits16(a, dtype):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).view(dtype)


def make_pool(L, NB, bs, H, D, dtype, seed, fill=None):
    g = torch.Generator().manual_seed(seed)
    if fill is not None:
        return [torch.full((2, NB, bs, H, D), fill, dtype=dtype) for _ in range(L)]
    return [torch.randn((2, NB, bs, H, D), generator=g).to(dtype) for _ in range(L)]


# ---------------------------------------------------------------- pack / unpack
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_pack_three_statements_agree(dtype):
    L, NB, bs, H, D = 2, 7, 2, 2, 3
    pool = make_pool(L, NB, bs, H, D, dtype, 0)
    idx = [5, 0, 3]
    ref = orc.ref_extract_kv_blocks(pool, idx)
    assert ref.shape == (L, 2, 3, bs, H, D) and ref.is_contiguous()
    brute = orc.brute_pack(pool, idx)
    c = orc.c_kv_pack(pool, idx)
    assert torch.equal(ref, brute)
    assert c.tobytes() == ref.numpy().tobytes() if dtype != torch.bfloat16 else \
        c.tobytes() == bits16(ref).tobytes()


def test_pack_is_index_select():
    pool = make_pool(3, 9, 2, 2, 4, torch.float16, 1)
    idx = torch.tensor([8, 1, 4, 2])
    closed = torch.stack([torch.index_select(p, 1, idx) for p in pool], 0)
    assert torch.equal(orc.ref_extract_kv_blocks(pool, idx.tolist()), closed)
    assert closed.numel() * closed.element_size() == 3 * 2 * 4 * (2 * 2 * 4 * 2)


def test_unpack_three_statements_agree_and_canary():
    L, NB, bs, H, D = 2, 8, 2, 2, 3
    g = torch.Generator().manual_seed(2)
    data = torch.randn((L, 2, 3, bs, H, D), generator=g).to(torch.float16)
    idx = [6, 1, 2]
    pools = [make_pool(L, NB, bs, H, D, torch.float16, 0, fill=-7.0) for _ in range(3)]
    orc.ref_write_kv_blocks(pools[0], idx, data)
    orc.brute_unpack(pools[1], idx, data)
    orc.c_kv_unpack(pools[2], idx, data)
    for l in range(L):
        assert torch.equal(pools[0][l], pools[1][l])
        assert torch.equal(pools[0][l], pools[2][l])
        untouched = [b for b in range(NB) if b not in idx]
        assert (pools[0][l][:, untouched] == -7.0).all()
        for j, b in enumerate(idx):
            assert torch.equal(pools[0][l][:, b], data[l, :, j])


def test_write_kv_blocks_count_mismatch_asserts():
    pool = make_pool(1, 4, 2, 1, 2, torch.float16, 0)
    with pytest.raises(AssertionError, match="Block count mismatch"):
        orc.ref_write_kv_blocks(pool, [0, 1], torch.zeros((1, 2, 3, 2, 1, 2), dtype=torch.float16))


def test_pack_unpack_roundtrip_under_other_table():
    L, NB = 3, 16
    src = make_pool(L, NB, 2, 2, 4, torch.bfloat16, 3)
    dst = make_pool(L, NB, 2, 2, 4, torch.bfloat16, 0, fill=1.5)
    g = torch.Generator().manual_seed(4)
    si = torch.randperm(NB, generator=g)[:6].tolist()
    di = torch.randperm(NB, generator=g)[:6].tolist()
    buf = orc.c_kv_pack(src, si)
    orc.c_kv_unpack(dst, di, buf)
    for l in range(L):
        for s, d in zip(si, di):
            assert torch.equal(dst[l][:, d], src[l][:, s])
        rest = [b for b in range(NB) if b not in di]
        assert (dst[l][:, rest] == 1.5).all()


def test_c_pack_skips_negative_and_oob_ids():
    pool = make_pool(1, 4, 1, 1, 4, torch.float16, 5)
    out = orc.c_kv_pack(pool, [2, -1, 9, 0])
    ref = orc.ref_extract_kv_blocks(pool, [2, 0])
    assert out[:, :, 0].tobytes() == ref[:, :, 0].numpy().tobytes()
    assert out[:, :, 3].tobytes() == ref[:, :, 1].numpy().tobytes()
    assert not out[:, :, 1].any() and not out[:, :, 2].any()


def test_pool6d_and_vision_forms_match_list_form():
    L, NB, bs, H, D = 2, 6, 2, 2, 3
    g = torch.Generator().manual_seed(6)
    pool6 = torch.randn((L, 2, NB, bs, H, D), generator=g).to(torch.float16)
    idx = [4, 0, 5]
    flat = orc.ref_pool6d_gather(pool6, idx)
    assert torch.equal(flat, orc.ref_extract_kv_blocks(list(pool6.unbind(0)), idx).flatten())
    dst6 = torch.zeros_like(pool6)
    orc.ref_pool6d_scatter(dst6, [1, 2, 3], flat)
    lst = list(torch.zeros_like(pool6).unbind(0))
    orc.ref_write_kv_blocks(lst, [1, 2, 3], flat.view(L, 2, 3, bs, H, D))
    assert torch.equal(dst6, torch.stack(lst, 0))
    ve = torch.randn((5, 3, 4), generator=g)
    got = orc.ref_vision_gather(ve, [3, 1])
    assert torch.equal(got, ve[[3, 1]])
    ve2 = torch.zeros_like(ve)
    orc.ref_vision_scatter(ve2, [0, 4], got)
    assert torch.equal(ve2[0], ve[3]) and torch.equal(ve2[4], ve[1]) and not ve2[1:4].any()


# ---------------------------------------------------------------- append
def test_reshape_and_cache_three_statements_and_slot_decomposition():
    NB, bs, H, D, T = 5, 4, 2, 3, 7
    g = torch.Generator().manual_seed(7)
    key = torch.randn((T, H, D), generator=g).to(torch.float16)
    value = torch.randn((T, H, D), generator=g).to(torch.float16)
    slots = torch.tensor([17, 3, -1, 0, 19, -1, 8])
    caches = []
    for fn in (orc.ref_reshape_and_cache_flash, orc.c_reshape_and_cache, orc.brute_reshape_and_cache):
        kc = torch.full((NB, bs, H, D), 9.0, dtype=torch.float16)
        vc = torch.full((NB, bs, H, D), 11.0, dtype=torch.float16)
        fn(key, value, kc, vc, slots)
        caches.append((kc, vc))
    for kc, vc in caches[1:]:
        assert torch.equal(kc, caches[0][0]) and torch.equal(vc, caches[0][1])
    kc, vc = caches[0]
    assert torch.equal(kc[4, 1], key[0])  # slot 17, bs 4 -> block 4, offset 1
    assert torch.equal(vc[4, 3], value[4])
    written = {17, 3, 0, 19, 8}
    for s in range(NB * bs):
        if s not in written:
            assert (kc.view(-1, H, D)[s] == 9.0).all() and (vc.view(-1, H, D)[s] == 11.0).all()


def test_reshape_and_cache_identity_slots_is_reshape():
    NB, bs, H, D = 3, 4, 2, 2
    T = NB * bs
    g = torch.Generator().manual_seed(8)
    key = torch.randn((T, H, D), generator=g).to(torch.bfloat16)
    value = torch.randn((T, H, D), generator=g).to(torch.bfloat16)
    kc = torch.zeros((NB, bs, H, D), dtype=torch.bfloat16)
    vc = torch.zeros_like(kc)
    orc.c_reshape_and_cache(key, value, kc, vc, torch.arange(T))
    assert torch.equal(kc, key.reshape(NB, bs, H, D)) and torch.equal(vc, value.reshape(NB, bs, H, D))


def test_reshape_and_cache_all_padding_leaves_cache():
    kc = torch.full((2, 2, 1, 4), 2.0, dtype=torch.float16)
    vc = torch.full((2, 2, 1, 4), 4.0, dtype=torch.float16)
    key = torch.ones((3, 1, 4), dtype=torch.float16)
    orc.c_reshape_and_cache(key, key, kc, vc, torch.tensor([-1, -1, -1]))
    orc.ref_reshape_and_cache_flash(key, key, kc, vc, torch.tensor([-1, -1, -1]))
    assert (kc == 2.0).all() and (vc == 4.0).all()


# ---------------------------------------------------------------- append, paged-attention layout
def _paged_caches(NB, H, D, bs, dtype, x=None):
    x = x or 16 // torch.empty((), dtype=dtype).element_size()
    kc = (torch.arange(NB * H * D * bs, dtype=torch.float32) % 61).to(dtype).view(NB, H, D // x, bs, x).clone()
    vc = (torch.arange(NB * H * D * bs, dtype=torch.float32) % 59).to(dtype).view(NB, H, D, bs).clone()
    return kc, vc


def test_paged_append_three_statements_agree():
    NB, bs, H, D, T = 4, 4, 2, 16, 9
    g = torch.Generator().manual_seed(17)
    key = torch.randn((T, H, D), generator=g).to(torch.float16)
    value = torch.randn((T, H, D), generator=g).to(torch.float16)
    slots = torch.tensor([13, 2, -1, 0, 15, -1, 8, 9, 5])
    outs = []
    for fn in (orc.ref_reshape_and_cache_paged, orc.c_reshape_and_cache_paged, orc.brute_reshape_and_cache_paged):
        kc, vc = _paged_caches(NB, H, D, bs, torch.float16)
        fn(key, value, kc, vc, slots)
        outs.append((kc, vc))
    for kc, vc in outs[1:]:
        assert torch.equal(kc, outs[0][0]) and torch.equal(vc, outs[0][1])
    kc, vc = outs[0]
    # slot 13, bs 4 -> block 3, offset 1; element d = 11 of head 1 sits in group 1 at position 3
    assert kc[3, 1, 1, 1, 3] == key[0, 1, 11] and vc[3, 1, 11, 1] == value[0, 1, 11]
    k0, v0 = _paged_caches(NB, H, D, bs, torch.float16)
    untouched = sorted(set(range(NB * bs)) - {13, 2, 0, 15, 8, 9, 5})
    for s in untouched:
        assert torch.equal(kc[s // bs, :, :, s % bs], k0[s // bs, :, :, s % bs])
        assert torch.equal(vc[s // bs, :, :, s % bs], v0[s // bs, :, :, s % bs])


def test_paged_append_identity_slots_is_a_permute():
    """slot = arange: the caches are the [NB, bs, H, D] reshape of the inputs with the token axis
    moved inwards (a statement that uses no index arithmetic at all)."""
    NB, bs, H, D, x = 3, 8, 2, 16, 8
    T = NB * bs
    g = torch.Generator().manual_seed(18)
    key = torch.randn((T, H, D), generator=g).to(torch.bfloat16)
    value = torch.randn((T, H, D), generator=g).to(torch.bfloat16)
    for fn in (orc.c_reshape_and_cache_paged, orc.ref_reshape_and_cache_paged):
        kc = torch.zeros((NB, H, D // x, bs, x), dtype=torch.bfloat16)
        vc = torch.zeros((NB, H, D, bs), dtype=torch.bfloat16)
        fn(key, value, kc, vc, torch.arange(T))
        assert torch.equal(kc, key.view(NB, bs, H, D // x, x).permute(0, 2, 3, 1, 4))
        assert torch.equal(vc, value.view(NB, bs, H, D).permute(0, 2, 3, 1))


def test_paged_append_equals_flash_append_then_permute():
    """Any slot table: appending in the flash layout (pinned above) and permuting the whole cache
    gives the paged caches."""
    NB, bs, H, D, x, T = 6, 4, 3, 8, 8, 11
    g = torch.Generator().manual_seed(19)
    key = torch.randn((T, H, D), generator=g).to(torch.float16)
    value = torch.randn((T, H, D), generator=g).to(torch.float16)
    slots = torch.randperm(NB * bs, generator=g)[:T].clone()
    slots[3] = -1
    kf = torch.randn((NB, bs, H, D), generator=g).to(torch.float16)
    vf = torch.randn((NB, bs, H, D), generator=g).to(torch.float16)
    kc = kf.view(NB, bs, H, D // x, x).permute(0, 2, 3, 1, 4).contiguous()
    vc = vf.permute(0, 2, 3, 1).contiguous()
    orc.c_reshape_and_cache(key, value, kf, vf, slots)
    orc.c_reshape_and_cache_paged(key, value, kc, vc, slots)
    assert torch.equal(kc, kf.view(NB, bs, H, D // x, x).permute(0, 2, 3, 1, 4))
    assert torch.equal(vc, vf.permute(0, 2, 3, 1))


def test_paged_append_fp8_is_cast_then_same_placement():
    NB, bs, H, D, x, T = 3, 4, 2, 32, 16, 10
    g = torch.Generator().manual_seed(20)
    key = (torch.randn((T, H, D), generator=g) * 3).to(torch.bfloat16)
    value = (torch.randn((T, H, D), generator=g) * 200).to(torch.bfloat16)  # some values overflow to NaN
    slots = torch.tensor([11, 10, -1, 0, 1, 2, 3, 7, 5, -1])
    ks, vs = 0.037, 0.5
    res = []
    for which in ("ref", "c"):
        kc = torch.full((NB, H, D // x, bs, x), 0x11, dtype=torch.uint8)
        vc = torch.full((NB, H, D, bs), 0x22, dtype=torch.uint8)
        if which == "ref":
            orc.ref_reshape_and_cache_paged(key, value, kc, vc, slots, "fp8", torch.tensor(ks), torch.tensor(vs))
        else:
            orc.c_reshape_and_cache_paged(key, value, kc, vc, slots, ks, vs)
        res.append((kc, vc))
    assert torch.equal(res[0][0], res[1][0]) and torch.equal(res[0][1], res[1][1])
    q = torch.from_numpy(orc.c_quant_fp8(value, vs))
    assert torch.equal(res[1][1][2, :, :, 3], q[0])  # slot 11 -> block 2, offset 3
    assert (res[1][1] == 0x7F).any() or (res[1][1] == 0xFF).any()


def test_golden_paged_small(golden_dir):
    z = np.load(os.path.join(golden_dir, "paged_small.npz"))
    bf = torch.bfloat16
    key, value = from_bits16(z["key"], bf), from_bits16(z["value"], bf)
    for fn in (orc.c_reshape_and_cache_paged, orc.ref_reshape_and_cache_paged):
        kc, vc = from_bits16(z["key_cache_before"], bf), from_bits16(z["value_cache_before"], bf)
        fn(key, value, kc, vc, torch.from_numpy(z["slots"]))
        assert bits16(kc).tobytes() == z["key_cache_after"].tobytes()
        assert bits16(vc).tobytes() == z["value_cache_after"].tobytes()


# ---------------------------------------------------------------- copy_blocks
def test_copy_blocks_three_statements_and_sources_unchanged():
    L, NB = 2, 10
    base = make_pool(L, NB, 2, 1, 4, torch.float16, 9)
    mapping = [(1, 7), (4, 0), (9, 2)]
    a = [p.clone() for p in base]
    b = [p.clone() for p in base]
    c = [p.clone() for p in base]
    orc.ref_copy_blocks(a, torch.tensor(mapping))
    orc.brute_copy_blocks(b, mapping)
    orc.c_copy_blocks(c, mapping)
    for l in range(L):
        assert torch.equal(a[l], b[l]) and torch.equal(a[l], c[l])
        for s, d in mapping:
            assert torch.equal(a[l][:, d], base[l][:, s])
            assert torch.equal(a[l][:, s], base[l][:, s])
        rest = [x for x in range(NB) if x not in (7, 0, 2)]
        assert torch.equal(a[l][:, rest], base[l][:, rest])


def test_concat_rows():
    g = torch.Generator().manual_seed(10)
    segs = [torch.randn((r, 5), generator=g).to(torch.bfloat16) for r in (2, 4, 1)]
    ref = orc.ref_concat_rows(segs)
    assert ref.shape == (7, 5)
    assert orc.c_concat_rows(segs).tobytes() == bits16(ref).tobytes()
    assert orc.ref_concat_rows(segs[:1]) is segs[0]


# ---------------------------------------------------------------- golden vectors
def test_golden_kv_small(golden_dir):
    z = np.load(os.path.join(golden_dir, "kv_small.npz"))
    f16 = torch.float16
    src = [from_bits16(a, f16) for a in z["src"]]
    si, di = z["src_idx"].tolist(), z["dst_idx"].tolist()
    packed = orc.c_kv_pack(src, si)
    assert packed.tobytes() == z["packed"].tobytes()
    assert bits16(orc.ref_extract_kv_blocks(src, si)).tobytes() == z["packed"].tobytes()
    dst = [torch.full_like(p, -7.0) for p in src]
    orc.c_kv_unpack(dst, di, packed)
    assert np.stack([bits16(p) for p in dst]).tobytes() == z["dst_after"].tobytes()
    key, value = from_bits16(z["key"], f16), from_bits16(z["value"], f16)
    NB, bs, H, D = z["key_cache_after"].shape
    kc = torch.full((NB, bs, H, D), 3.0, dtype=f16)
    vc = torch.full((NB, bs, H, D), 5.0, dtype=f16)
    orc.c_reshape_and_cache(key, value, kc, vc, z["slots"])
    assert bits16(kc).tobytes() == z["key_cache_after"].tobytes()
    assert bits16(vc).tobytes() == z["value_cache_after"].tobytes()
    cb = [p.clone() for p in src]
    orc.c_copy_blocks(cb, z["mapping"])
    assert np.stack([bits16(p) for p in cb]).tobytes() == z["copy_after"].tobytes()
    segs = [from_bits16(z[f"seg{i}"], torch.bfloat16) for i in range(3)]
    assert orc.c_concat_rows(segs).tobytes() == z["cat"].tobytes()


# ---------------------------------------------------------------- fp8
KAT_IN = [448, 464, 465, 480, -1000, 2 ** -9, 2 ** -10, 2 ** -10 * 1.0001, 17, 18, 19, float("inf")]
KAT_OUT = [126, 126, 127, 127, 255, 1, 0, 1, 88, 89, 90, 127]


def test_fp8_known_answers():
    lib = orc.lib()
    got = [lib.orc_f32_to_e4m3fn(np.float32(x)) for x in KAT_IN]
    assert got == KAT_OUT
    assert lib.orc_f32_to_e4m3fn(np.float32("nan")) & 0x7F == 0x7F
    assert lib.orc_f32_to_e4m3fn(np.float32(-0.0)) == 0x80
    assert lib.orc_f32_to_e4m3fn(np.float32(-(2.0 ** -11))) == 0x80
    assert lib.orc_f32_to_e4m3fn(np.float32(2.0 ** -6)) == 0x08  # smallest normal


def test_fp8_golden_special_values(golden_dir):
    kat = json.load(open(os.path.join(golden_dir, "fp8_kat.json")))
    xs = np.array(kat["special_inputs_f32_bits"], dtype=np.int32).view(np.float32)
    lib = orc.lib()
    got = [lib.orc_f32_to_e4m3fn(x) for x in xs]
    assert got == kat["special_bytes"]
    assert kat["special_bytes"][:12] == KAT_OUT


def test_fp8_decode_table_is_the_format_definition():
    lib = orc.lib()
    tq = torch.arange(256, dtype=torch.int32).to(torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    for b in range(256):
        v = lib.orc_e4m3fn_to_f32(b)
        s, e, m = b >> 7, (b >> 3) & 15, b & 7
        if e == 15 and m == 7:
            assert np.isnan(v) and np.isnan(tq[b])
            continue
        want = (m / 8.0) * 2.0 ** -6 if e == 0 else (1 + m / 8.0) * 2.0 ** (e - 7)
        want = -want if s else want
        assert v == np.float32(want) and v == tq[b]
        # every representable value encodes back to its own byte
        assert lib.orc_f32_to_e4m3fn(np.float32(v)) == b


@pytest.mark.parametrize("dtype,name", [(torch.bfloat16, "bf16"), (torch.float16, "f16")])
def test_fp8_quant_exhaustive_vs_torch_cast(golden_dir, dtype, name):
    kat = json.load(open(os.path.join(golden_dir, "fp8_kat.json")))
    allx = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(dtype)
    for s in kat["scales"]:
        got = orc.c_quant_fp8(allx, s)
        want = (allx.float() / torch.tensor(s, dtype=torch.float32)).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, f"scale {s}: first mismatch at bits {bad[:5]}: {got[bad[:5]]} vs {want[bad[:5]]}"
        assert hashlib.sha256(got.tobytes()).hexdigest() == kat["sweep_sha256"][f"{name}@{s}"]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fp8_saturating_quant_exhaustive_vs_torch_clamp_cast(golden_dir, dtype):
    """The saturating mode is pinned to the library routines that define it — torch.clamp then
    torch's cast — on every 16-bit input, and to the non-saturating cast (pinned above) wherever
    that one does not overflow. A wrong clamp bound, a clamp after the cast, or NaN folded into
    the bound each fail one of the three checks."""
    kat = json.load(open(os.path.join(golden_dir, "fp8_kat.json")))
    allx = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(dtype)
    nan_in = torch.isnan(allx.float()).numpy()
    for s in kat["scales"]:
        got = orc.c_quant_fp8_sat(allx, s)
        want = orc.ref_quant_fp8_sat(allx, s).numpy()
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, f"scale {s}: first mismatch at bits {bad[:5]}: {got[bad[:5]]} vs {want[bad[:5]]}"
        plain = orc.c_quant_fp8(allx, s)
        finite = (plain & 0x7F) != 0x7F
        assert (got[finite] == plain[finite]).all()            # no overflow: the two modes agree
        over = ~finite & ~nan_in
        assert ((got[over] & 0x7F) == 0x7E).all()              # overflow and +-inf: 448 with the sign
        assert (got[over] & 0x80 == plain[over] & 0x80).all()
        assert ((got[nan_in] & 0x7F) == 0x7F).all()            # NaN stays NaN


def test_fp8_saturating_known_answers():
    x = torch.tensor([448.0, 464.0, 465.0, 1.0e6, float("inf"), -465.0, -float("inf"), float("nan"), 17.0, 2.0 ** -10],
                     dtype=torch.float32).to(torch.bfloat16)
    got = orc.c_quant_fp8_sat(x, 1.0).tolist()
    assert got[:7] == [0x7E, 0x7E, 0x7E, 0x7E, 0x7E, 0xFE, 0xFE]
    assert got[7] & 0x7F == 0x7F and got[8:] == [88, 0]
    # a scale turns the bound into 448 * scale in input units
    assert orc.c_quant_fp8_sat(torch.tensor([44.0, 44.8, 50.0], dtype=torch.bfloat16), 0.1).tolist()[1:] == [0x7E, 0x7E]


def test_fp8_monotone_and_nearest():
    """Brute force from the definition: the chosen code is a nearest representable
    value (ties to the even code), for a dense sample of magnitudes below 464."""
    lib = orc.lib()
    reps = np.array([lib.orc_e4m3fn_to_f32(b) for b in range(0x7F)], dtype=np.float64)  # 0 .. 448, increasing
    assert (np.diff(reps) > 0).all()
    rng = np.random.default_rng(0)
    xs = np.concatenate([rng.uniform(0, 464, 4000), rng.uniform(0, 0.05, 2000),
                         (reps[:-1] + reps[1:]) / 2]).astype(np.float32)
    for x in xs:
        if x >= 464:
            continue
        b = lib.orc_f32_to_e4m3fn(x)
        d = np.abs(reps - np.float64(x))
        best = d.min()
        assert abs(reps[b] - np.float64(x)) == best
        ties = np.nonzero(d == best)[0]
        if ties.size == 2:
            assert b % 2 == 0


def test_fp8_dequant_exhaustive(golden_dir):
    kat = json.load(open(os.path.join(golden_dir, "fp8_kat.json")))
    allq = np.arange(256, dtype=np.uint8)
    tq = torch.from_numpy(allq).view(torch.float8_e4m3fn).float()
    for s in kat["scales"]:
        got = orc.c_dequant_fp8(allq, s, torch.bfloat16)
        prod = tq * torch.tensor(s, dtype=torch.float32)
        want = bits16(prod.to(torch.bfloat16)).copy()
        nan = np.isnan(prod.numpy())
        assert (got[nan] == 0x7FC0).all()
        assert (got[~nan] == want[~nan]).all()
        if f"bf16@{s}" in kat["dequant"]:
            assert got.tolist() == kat["dequant"][f"bf16@{s}"]
        got16 = orc.c_dequant_fp8(allq, s, torch.float16)
        want16 = bits16(prod.to(torch.float16)).copy()
        assert (got16[nan] == 0x7E00).all()
        assert (got16[~nan] == want16[~nan]).all()


def test_f32_to_16bit_roundings_exhaustive_high_halves():
    """bf16 / f16 RNE of the C oracle against torch casts on a structured sweep:
    every 16-bit high half combined with low halves that hit below / at / above the tie."""
    lib = orc.lib()
    hi = np.arange(65536, dtype=np.uint32) << 16
    for low in (0x0000, 0x7FFF, 0x8000, 0x8001, 0xFFFF):
        f = torch.from_numpy((hi | low).view(np.int32)).view(torch.float32)
        want = bits16(f.to(torch.bfloat16))
        fn = f.numpy()
        got = np.array([lib.orc_f32_to_bf16(v) for v in fn[::37]], dtype=np.uint16)
        w = want[::37].copy()
        nan = np.isnan(fn[::37])
        assert (got[~nan] == w[~nan]).all() and (got[nan] == 0x7FC0).all()
    g = torch.Generator().manual_seed(11)
    x = torch.cat([torch.randn(4000, generator=g) * 100, torch.randn(2000, generator=g) * 1e-6,
                   torch.tensor([65504.0, 65519.9, 65520.0, 1e9, -1e9, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.001, 0.0, -0.0])])
    want = bits16(x.to(torch.float16))
    got = np.array([lib.orc_f32_to_f16(v) for v in x.numpy()], dtype=np.uint16)
    assert (got == want).all()


def test_fp8_append_and_dequant_unpack_compose():
    NB, bs, H, D, T = 4, 2, 2, 8, 6
    g = torch.Generator().manual_seed(12)
    key = (torch.randn((T, H, D), generator=g) * 3).to(torch.bfloat16)
    value = (torch.randn((T, H, D), generator=g) * 3).to(torch.bfloat16)
    slots = torch.tensor([5, -1, 0, 7, 2, -1])
    ks, vs = 0.05, 0.02
    kc = torch.full((NB, bs, H, D), 0x11, dtype=torch.uint8)
    vc = torch.full((NB, bs, H, D), 0x22, dtype=torch.uint8)
    orc.c_reshape_and_cache_fp8(key, value, kc, vc, slots, ks, vs)
    kc2 = torch.full((NB, bs, H, D), 0x11, dtype=torch.uint8)
    vc2 = torch.full((NB, bs, H, D), 0x22, dtype=torch.uint8)
    orc.ref_reshape_and_cache_flash(key, value, kc2.view(torch.float8_e4m3fn), vc2.view(torch.float8_e4m3fn), slots,
                                    "fp8", torch.tensor(ks), torch.tensor(vs))
    assert torch.equal(kc, kc2) and torch.equal(vc, vc2)
    assert (kc.view(-1, H * D)[[1, 3, 4, 6]] == 0x11).all()
    # dequantising unpack of those bytes into a bf16 pool
    pool_fp8 = [torch.stack([kc, vc], 0)]
    idx = [2, 0, 3]
    packed = orc.c_kv_pack(pool_fp8, idx)
    a = [torch.zeros((2, NB, bs, H, D), dtype=torch.bfloat16)]
    b = [torch.zeros((2, NB, bs, H, D), dtype=torch.bfloat16)]
    dst_idx = [1, 3, 0]
    orc.c_unpack_dequant_fp8(a, dst_idx, packed, [ks], [vs])
    orc.ref_unpack_dequant_fp8(b, dst_idx, torch.from_numpy(packed), torch.tensor([ks]), torch.tensor([vs]))
    na = torch.isnan(a[0].float())
    assert torch.equal(na, torch.isnan(b[0].float()))
    assert torch.equal(torch.where(na, torch.zeros_like(a[0]), a[0]), torch.where(na, torch.zeros_like(b[0]), b[0]))

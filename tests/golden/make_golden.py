"""Generates the committed fixtures of tests/golden/ with stock torch on the CPU.

Nothing from /root/reference is imported or executed: the reference's path is a
handful of torch indexing expressions (cited in oracle/kv_oracle.py) and one
library cast, ``Tensor.to(torch.float8_e4m3fn)``; both are evaluated here with
the torch that ships in this image and frozen as data.

    python tests/golden/make_golden.py

writes
    kv_small.npz     seeded tiny pools, block tables, slot mapping and the
                     expected results of pack / unpack / append / copy_blocks /
                     concat (raw little-endian bit patterns as uint16 / uint8)
    paged_small.npz  an append into the paged-attention layout, stated as a flat-slot
                     index_copy followed by a permute of the whole cache (not as an
                     indexed assignment into the transposed layout)
    fp8_kat.json     known answers of the fp8-e4m3fn cast: the explicit vector of
                     special values and the SHA-256 of the exhaustive sweep of
                     all 65 536 bf16 (and f16) bit patterns at several scales,
                     plus the full dequantisation table for three scales
"""
import hashlib
import json
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
SCALES = [0.01, 0.037, 0.1, 1.0, 0.0625, 0.07321]


def bits16(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def kv_small():
    g = torch.Generator().manual_seed(1234)
    L, NB, bs, H, D = 3, 11, 2, 2, 8
    src = [torch.randn((2, NB, bs, H, D), generator=g).to(torch.float16) for _ in range(L)]
    dst = [torch.full((2, NB, bs, H, D), -7.0, dtype=torch.float16) for _ in range(L)]
    src_idx = torch.randperm(NB, generator=g)[:5]
    dst_idx = torch.randperm(NB, generator=g)[:5]
    # pack: worker.py:597-608
    packed = torch.stack([p[:, src_idx, :, :, :] for p in src], dim=0)
    # unpack under another table: worker.py:628-633
    for l, p in enumerate(dst):
        p[:, dst_idx, :, :, :] = packed[l]
    # append: flat-slot index_copy with slot >= 0
    T = 9
    key = torch.randn((T, H, D), generator=g).to(torch.float16)
    value = torch.randn((T, H, D), generator=g).to(torch.float16)
    slots = torch.randperm(NB * bs, generator=g)[:T].clone()
    slots[2] = -1
    slots[7] = -1
    kc = torch.full((NB, bs, H, D), 3.0, dtype=torch.float16)
    vc = torch.full((NB, bs, H, D), 5.0, dtype=torch.float16)
    valid = slots >= 0
    kc.view(NB * bs, H, D).index_copy_(0, slots[valid], key[valid])
    vc.view(NB * bs, H, D).index_copy_(0, slots[valid], value[valid])
    # copy_blocks: pairs with disjoint destinations
    cb = [p.clone() for p in src]
    perm = torch.randperm(NB, generator=g)
    mapping = torch.stack([perm[:4], perm[4:8]], dim=1)
    for p in cb:
        p[:, mapping[:, 1]] = p[:, mapping[:, 0]]
    # ragged concat
    segs = [torch.randn((r, 6), generator=g).to(torch.bfloat16) for r in (3, 1, 4)]
    cat = torch.cat(segs, 0)
    np.savez_compressed(
        os.path.join(HERE, "kv_small.npz"),
        src=np.stack([bits16(p) for p in src]), src_idx=src_idx.numpy(), dst_idx=dst_idx.numpy(),
        packed=bits16(packed), dst_after=np.stack([bits16(p) for p in dst]),
        key=bits16(key), value=bits16(value), slots=slots.numpy(),
        key_cache_after=bits16(kc), value_cache_after=bits16(vc),
        mapping=mapping.numpy(), copy_after=np.stack([bits16(p) for p in cb]),
        seg0=bits16(segs[0]), seg1=bits16(segs[1]), seg2=bits16(segs[2]), cat=bits16(cat),
    )


def paged_small():
    g = torch.Generator().manual_seed(4321)
    NB, bs, H, D, x, T = 5, 4, 2, 16, 8, 13
    key = torch.randn((T, H, D), generator=g).to(torch.bfloat16)
    value = torch.randn((T, H, D), generator=g).to(torch.bfloat16)
    slots = torch.randperm(NB * bs, generator=g)[:T].clone()
    slots[4] = -1
    slots[11] = -1
    # fill values differ per position so that a transposed write into the wrong place shows
    kflat = (torch.arange(NB * bs * H * D, dtype=torch.float32) % 251).to(torch.bfloat16).view(NB * bs, H, D)
    vflat = (torch.arange(NB * bs * H * D, dtype=torch.float32) % 241).to(torch.bfloat16).view(NB * bs, H, D)
    k_before = kflat.view(NB, bs, H, D // x, x).permute(0, 2, 3, 1, 4).contiguous()
    v_before = vflat.view(NB, bs, H, D).permute(0, 2, 3, 1).contiguous()
    valid = slots >= 0
    kflat = kflat.clone().index_copy_(0, slots[valid], key[valid])
    vflat = vflat.clone().index_copy_(0, slots[valid], value[valid])
    k_after = kflat.view(NB, bs, H, D // x, x).permute(0, 2, 3, 1, 4).contiguous()
    v_after = vflat.view(NB, bs, H, D).permute(0, 2, 3, 1).contiguous()
    np.savez_compressed(os.path.join(HERE, "paged_small.npz"), key=bits16(key), value=bits16(value),
                        slots=slots.numpy(), key_cache_before=bits16(k_before), value_cache_before=bits16(v_before),
                        key_cache_after=bits16(k_after), value_cache_after=bits16(v_after))


def fp8_kat():
    special = [448, 464, 465, 480, -1000, 2 ** -9, 2 ** -10, 2 ** -10 * 1.0001, 17, 18, 19, float("inf"),
               float("-inf"), float("nan"), -0.0, 0.0, -2 ** -11, 479.9, 1e-40, 0.5, -1.75, 2 ** -6, 2 ** -7 * 1.9]
    sp = torch.tensor(special, dtype=torch.float32)
    sp_bytes = sp.to(torch.float8_e4m3fn).view(torch.uint8).tolist()
    out = {"special_inputs_f32_bits": sp.view(torch.int32).tolist(), "special_bytes": sp_bytes,
           "scales": SCALES, "sweep_sha256": {}, "dequant": {}}
    for name, dt in (("bf16", torch.bfloat16), ("f16", torch.float16)):
        allx = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(dt)
        for s in SCALES:
            q = (allx.float() / torch.tensor(s, dtype=torch.float32)).to(torch.float8_e4m3fn).view(torch.uint8)
            out["sweep_sha256"][f"{name}@{s}"] = hashlib.sha256(q.numpy().tobytes()).hexdigest()
    allq = torch.arange(256, dtype=torch.int32).to(torch.uint8).view(torch.float8_e4m3fn).float()
    for s in SCALES[:3]:
        # scalar c10 rule for NaN -> 0x7FC0 (torch's vectorised CPU path gives 0xFFFF instead)
        d = (allq * torch.tensor(s, dtype=torch.float32))
        b = d.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16).copy()
        b[np.isnan(d.numpy())] = 0x7FC0
        out["dequant"][f"bf16@{s}"] = b.tolist()
    with open(os.path.join(HERE, "fp8_kat.json"), "w") as f:
        json.dump(out, f)


if __name__ == "__main__":
    kv_small()
    paged_small()
    fp8_kat()
    print("wrote", sorted(os.listdir(HERE)))

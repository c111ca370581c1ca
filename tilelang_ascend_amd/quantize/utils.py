"""Weight preparation helpers of tilelang/quantize/utils.py, vectorised on torch tensors.

These run offline (once per checkpoint), on whatever device the tensors are on; the per-column
Python loops of the reference are replaced by whole-tensor shifts.
"""
from __future__ import annotations

import torch


def gen_quant4(k, n, groupsize=-1):
    """tilelang/quantize/utils.py:5-50: random fp16 weights [k, n], symmetric 4-bit quantisation per
    (group of `groupsize` rows, column): s = max|w| / 8, q = clamp(round(w / s) + 8, 0, 16) (the
    upper clamp is 16 in the reference, reached only by the +max element of a group).
    Returns (original_w, nn.Linear holding the dequantised weights, s [k/groupsize, n], q - 8)."""
    import torch.nn as nn

    maxq = 2**4
    w = torch.randn((k, n), dtype=torch.half, device="cpu")
    original_w = w.clone()
    if groupsize == -1:
        groupsize = k
    groups = k // groupsize
    wg = w.reshape(groups, groupsize, n)
    s = wg.abs().amax(dim=1, keepdim=True) * (2 / maxq)           # [groups, 1, n]
    q = torch.clamp(torch.round(wg / s).int() + maxq // 2, 0, maxq)
    ref = ((q - maxq // 2).half() * s).reshape(k, n).contiguous()
    linear = nn.Linear(k, n, bias=False)
    linear.weight.data = ref.t()
    return original_w, linear, s.reshape(groups, n).contiguous(), (q - maxq // 2).reshape(k, n).contiguous()


def general_compress(lowprecision_weight, source_bits=4, storage_dtype=None):
    """utils.py:53-69: pack `8 // source_bits` consecutive elements of the last dimension into one
    byte, element k of a byte at bit source_bits * k.  Like the reference the operands are not
    masked (pass values that fit in source_bits) and the byte is accumulated as int8."""
    if storage_dtype is None:
        storage_dtype = torch.int8
    epb = 8 // source_bits
    w = lowprecision_weight
    if w.dtype == torch.float16:
        w = w.to(torch.int8)
    n_out = w.shape[-1] // epb
    fields = w[..., : n_out * epb].reshape(*w.shape[:-1], n_out, epb).to(torch.int32)
    shifts = torch.arange(epb, device=w.device, dtype=torch.int32) * source_bits
    shifted = (fields << shifts) & 0xFF
    packed = shifted[..., 0]
    for j in range(1, epb):
        packed = packed | shifted[..., j]
    packed = torch.where(packed >= 128, packed - 256, packed).to(torch.int8)
    return packed.to(storage_dtype)


def interleave_weight(qweight, nbits=4, target_dtype="float16"):
    """utils.py:73-126: permute the `32 // nbits` fields of every 32-bit word so that one shift + mask
    per pair yields fields (i, i + 4) side by side in 16-bit (fp16) or 8-bit (int8) lanes:
    field i moves to bit (i % G) * stride + (i // G) * nbits, stride = 16 | 8, G = 32 // stride.
    For nbits = 4: order e0,e2,e4,e6,e1,e3,e5,e7 (fp16) and e0,e4,e1,e5,e2,e6,e3,e7 (int8)."""
    assert target_dtype in ["float16", "int8"]
    q = qweight.contiguous().view(torch.int32).to(torch.int64) & 0xFFFFFFFF
    stride = 8 if target_dtype == "int8" else 16
    mask = (1 << nbits) - 1
    G = 32 // stride
    per = stride // nbits
    new = torch.zeros_like(q)
    for off in range(G * per):
        shift = (off % G) * stride + (off // G) * nbits
        new |= ((q >> (nbits * off)) & mask) << shift

    # 1-bit sources, and 2-bit sources for the float16 target: the reference continues with masks written
    # torch.int32(0x...) (utils.py:103-124), which raises TypeError (a dtype object is not callable); a caller of
    # the reference never gets a value from these branches, and gets the same exception here.
    if nbits == 1 or (nbits == 2 and target_dtype == "float16"):
        raise TypeError(f"'torch.dtype' object is not callable (interleave_weight of {nbits}-bit weights for {target_dtype} "
                        "raises in the reference as well)")
    new = torch.where(new >= (1 << 31), new - (1 << 32), new).to(torch.int32)
    return new.view(torch.int8).reshape(qweight.shape)

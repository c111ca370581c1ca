"""On-disk form of repacked weights: what `general_compress` / `interleave_weight` / the quantisers produce
(tilelang/quantize/utils.py:53-126), kept so that the offline repacking runs once.

A file holds plain tensors and plain numbers only -- {"format", "B_packed", "scales", "zeros", "layout", "group",
"zero_scalar", "N", "K"} written with `torch.save` -- and is read back with `torch.load(weights_only=True)`, which
executes nothing from the file.  The reference keeps quantised weights as ordinary tensors of a checkpoint too; it has no
file format of its own for them.
"""
from __future__ import annotations

import torch

FORMAT = "tlq-w4-packed/1"
LAYOUTS = ("plain", "interleaved")


def save_packed(path, B_packed: torch.Tensor, scales=None, zeros=None, *, layout: str = "plain", group: int = 128) -> None:
    """B_packed: uint8 / int8 [N, K/2]; scales: [N, K/group] or None; zeros: [N, K/group] tensor, a number or None."""
    if layout not in LAYOUTS:
        raise ValueError(f"layout must be one of {LAYOUTS}, got {layout!r}")
    if B_packed.dim() != 2 or B_packed.dtype not in (torch.uint8, torch.int8):
        raise TypeError("B_packed must be a uint8 / int8 matrix [N, K/2]")
    N, K = B_packed.shape[0], B_packed.shape[1] * 2
    if group <= 0 or K % group != 0:
        raise ValueError(f"group={group} does not divide K={K}")
    for name, t in (("scales", scales), ("zeros", zeros)):
        if torch.is_tensor(t) and tuple(t.shape) != (N, K // group):
            raise ValueError(f"{name} must be [N, K/group] = {(N, K // group)}, got {tuple(t.shape)}")
    blob = {"format": FORMAT, "layout": layout, "group": int(group), "N": N, "K": K,
            "B_packed": B_packed.detach().cpu().contiguous(),
            "scales": scales.detach().cpu().contiguous() if torch.is_tensor(scales) else None,
            "zeros": zeros.detach().cpu().contiguous() if torch.is_tensor(zeros) else None,
            "zero_scalar": None if (zeros is None or torch.is_tensor(zeros)) else float(zeros)}
    torch.save(blob, path)


def load_packed(path, device=None) -> dict:
    """The dictionary save_packed wrote, tensors on `device` (default: as saved, on the host); `zeros` is the tensor,
    the number or None that was saved."""
    blob = torch.load(path, map_location="cpu", weights_only=True)
    if not isinstance(blob, dict) or blob.get("format") != FORMAT:
        raise ValueError(f"{path}: not a {FORMAT} file")
    if blob["layout"] not in LAYOUTS:
        raise ValueError(f"{path}: unknown layout {blob['layout']!r}")
    out = {"layout": blob["layout"], "group": int(blob["group"]), "N": int(blob["N"]), "K": int(blob["K"])}
    for name in ("B_packed", "scales", "zeros"):
        t = blob[name]
        out[name] = t.to(device) if (torch.is_tensor(t) and device is not None) else t
    if out["zeros"] is None and blob["zero_scalar"] is not None:
        out["zeros"] = float(blob["zero_scalar"])
    if tuple(out["B_packed"].shape) != (out["N"], out["K"] // 2):
        raise ValueError(f"{path}: B_packed has shape {tuple(out['B_packed'].shape)}, header says N={out['N']} K={out['K']}")
    return out

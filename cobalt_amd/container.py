"""CBK1 directories: `manifest.json` plus one `.bin` per decoder layer, each a concatenation of
256-byte aligned arrays that are, byte for byte, what the kernels read (reference:
docs/FORMAT.md:1-37 container, :126-151 fused matrices and `alias_of`; writer
src/cobaltkernel/pack_cobalt.py:390-505; loader src/cobaltkernel/runner.py:413-484).

Reading is offset-driven: every matrix entry of the manifest names its blob and the offset and
length of each of its arrays, so row-fused matrices and the `alias_of` entries that point into
them need no special case.  A layer's blob is loaded once; the PackedMatrix of every matrix in
it is a view (offset table) onto that one tensor.  On disk the rows are in the reference's
row-major order; `to_tiled()` reorders them for the decode kernel after the move to the GPU.
"""
from __future__ import annotations

import json
import os
from typing import Dict, List, Optional, Tuple

import numpy as np
import torch

from . import format as F

FORMAT_NAME = "CBK1"
FORMAT_VERSION = 1


def _entry(pm: F.PackedMatrix, blob_name: str, base: Dict[str, int]) -> dict:
    arrays = {}
    for name in ("data", "row_off", "scale", "zero", "col_scale"):
        if name in pm.offs and (name != "col_scale" or pm.cs_rows):
            arrays[name] = {"off": base[name], "bytes": int(pm.array(name).numel() * pm.array(name).element_size())}
    e = {"K": pm.K, "N": pm.N, "G": pm.G, "layout": pm.layout, "layout_name": F.LAYOUT_NAME[pm.layout],
         "cs_rows": pm.cs_rows, "n_survivors": pm.n_survivors, "stream_bytes": pm.stream_bytes(),
         "bpw": pm.bpw(), "blob": blob_name, "arrays": arrays}
    if pm.layout in (F.BLKC, F.DENSEB) or pm.group != 128:
        e.update(bits=pm.bits, group=pm.group, keep=pm.keep)       # the extension layouts carry their parameters
    if pm.cs_rows == 3:
        e["cs_splits"] = list(pm.cs_splits)
    return e


def write_container(path: str, layers: List[Dict[str, F.PackedMatrix]], config: Optional[dict] = None) -> dict:
    """Write `layers[i][name]` (row-major PackedMatrix objects) as layer_%02d.bin + manifest.json.
    Returns the manifest."""
    os.makedirs(path, exist_ok=True)
    manifest = {"format": FORMAT_NAME, "version": FORMAT_VERSION, "config": dict(config or {}), "layers": []}
    for li, mats in enumerate(layers):
        blob_name = f"layer_{li:02d}.bin"
        pos = 0
        entries = {}
        with open(os.path.join(path, blob_name), "wb") as f:
            for name, pm in mats.items():
                if pm.tiled:
                    raise ValueError(f"{name}: write the row-major order; the tiled order is a load-time transform")
                base = {}
                for an in ("data", "row_off", "scale", "zero", "col_scale"):
                    if an not in pm.offs or (an == "col_scale" and not pm.cs_rows):
                        continue
                    pad = F._align(pos, F.ARR_ALIGN) - pos
                    f.write(b"\0" * pad)
                    pos += pad
                    raw = pm.array(an).contiguous().view(torch.uint8).cpu().numpy().tobytes()
                    base[an] = pos
                    f.write(raw)
                    pos += len(raw)
                entries[name] = _entry(pm, blob_name, base)
            f.write(b"\0" * (F._align(pos, F.ARR_ALIGN) - pos))
        manifest["layers"].append(entries)
    with open(os.path.join(path, "manifest.json"), "w") as f:
        json.dump(manifest, f, indent=1)
    return manifest


def matrix_from_entry(e: dict, blob: torch.Tensor) -> F.PackedMatrix:
    """PackedMatrix view of one manifest entry onto its (already loaded) blob."""
    layout = int(e["layout"])
    bits, group, keep = F.canon(layout, e.get("bits"), e.get("group"), e.get("keep"))
    a = e["arrays"]
    offs = {k: int(v["off"]) for k, v in a.items()}
    K, N = int(e["K"]), int(e["N"])
    data_bytes = int(a["data"]["bytes"]) - F.BLOB_TAIL
    zero = blob[offs["zero"]: offs["zero"] + int(a["zero"]["bytes"])]
    flags = F.FLAG_ZERO_LE_128 if int(zero.max()) <= 128 else 0
    return F.PackedMatrix(blob, offs, K, N, layout, bits, group, keep, int(e.get("cs_rows", 0)),
                          tuple(e.get("cs_splits", (0, 0))), data_bytes, int(e.get("n_survivors", 0)), flags=flags)


def read_container(path: str, device="cpu", include_aliases: bool = True) -> Tuple[dict, List[Dict[str, F.PackedMatrix]]]:
    """(manifest, layers) with every blob read once and placed on `device`."""
    with open(os.path.join(path, "manifest.json")) as f:
        manifest = json.load(f)
    if manifest.get("format") != FORMAT_NAME:
        raise ValueError(f"{path}: not a {FORMAT_NAME} directory")
    blobs: Dict[str, torch.Tensor] = {}
    layers = []
    for entries in manifest["layers"]:
        mats = {}
        for name, e in entries.items():
            if e.get("alias_of") and not include_aliases:
                continue
            bn = e["blob"]
            if bn not in blobs:
                raw = np.fromfile(os.path.join(path, bn), dtype=np.uint8)
                blobs[bn] = torch.from_numpy(raw).to(device)
            mats[name] = matrix_from_entry(e, blobs[bn])
        layers.append(mats)
    return manifest, layers


def total_stream_bytes(manifest: dict) -> int:
    """Weight bytes one pass over the model streams; entries with `alias_of` are views into a
    fused matrix and are not counted twice (docs/FORMAT.md:146-151)."""
    return sum(int(e["stream_bytes"]) for entries in manifest["layers"] for e in entries.values()
               if not e.get("alias_of"))


def check_container(path: str, layers: int = 2, device="cpu", strict: bool = True) -> dict:
    """Structural and numerical check of a CBK1 directory, the role of the reference's
    `check_artifact` (src/prod/verify.py:64-152): every array lies inside its blob, the bytes per
    weight add up, and, for the first `layers` layers, every blocked matrix keeps exactly `keep`
    columns in every 32-column block.  With a GPU `device` the matrices are also dequantised by the
    library: all values finite, every pruned position exactly zero.  Returns a report with the
    list of `problems`; raises ValueError on any of them if `strict`."""
    with open(os.path.join(path, "manifest.json")) as f:
        man = json.load(f)
    problems: List[str] = []
    rep = {"path": path, "format": man.get("format"), "matrices": {}, "problems": problems}
    if man.get("format") != FORMAT_NAME:
        problems.append(f"format is {man.get('format')!r}, want {FORMAT_NAME!r}")
    sizes: Dict[str, int] = {}
    for li, entries in enumerate(man.get("layers", [])):
        for name, e in entries.items():
            bn = e["blob"]
            bp = os.path.join(path, bn)
            if bn not in sizes:
                if not os.path.exists(bp):
                    problems.append(f"missing blob {bn}")
                    sizes[bn] = -1
                else:
                    sizes[bn] = os.path.getsize(bp)
            if sizes[bn] < 0:
                continue
            for an, a in e["arrays"].items():
                if a["off"] % F.ARR_ALIGN:
                    problems.append(f"{bn}:{name}.{an} starts at {a['off']}, not on a {F.ARR_ALIGN}-byte boundary")
                if a["off"] + a["bytes"] > sizes[bn]:
                    problems.append(f"{bn}:{name}.{an} runs past the blob ({a['off']}+{a['bytes']} > {sizes[bn]})")
    rep["blob_bytes"] = sum(v for v in sizes.values() if v > 0)
    owned = [e for entries in man.get("layers", []) for e in entries.values() if not e.get("alias_of")]
    params = sum(e["K"] * e["N"] for e in owned)
    if params:
        rep["bpw"] = 8.0 * sum(e["stream_bytes"] for e in owned) / params
        want = sum(e["bpw"] * e["K"] * e["N"] for e in owned) / params
        if abs(rep["bpw"] - want) > 1e-6:
            problems.append(f"bytes per weight recompute to {rep['bpw']:.6f}, the entries say {want:.6f}")
    if not problems:
        on_gpu = torch.device(device).type == "cuda"
        _, mats_by_layer = read_container(path, device=device, include_aliases=False)
        for li, mats in enumerate(mats_by_layer[:layers]):
            for name, pm in mats.items():
                info = {"layout": F.LAYOUT_NAME[pm.layout], "shape": [pm.K, pm.N]}
                keep = None
                if pm.layout in (F.BLK1632_4, F.BLK1632_6, F.BLKC):
                    st = F.row_stride(pm.layout, pm.N, pm.bits, pm.group, pm.keep or None)
                    rows = pm.array("data")[: pm.K * st].view(pm.K, st)
                    keep = F.unpack_mask(rows[:, : pm.N // 8], pm.N)
                    cnt = keep.reshape(pm.K, pm.N // F.BLOCK, F.BLOCK).sum(-1)
                    lo, hi = int(cnt.min()), int(cnt.max())
                    info["block_survivors"] = [lo, hi]
                    if not lo == hi == pm.keep:
                        problems.append(f"layer {li} {name}: {lo}..{hi} survivors per 32-column block, want exactly {pm.keep}")
                if on_gpu:
                    from . import ops
                    W = ops.dequant(pm, torch.float32)
                    info["finite"] = bool(torch.isfinite(W).all())
                    info["zero_fraction"] = float((W == 0).float().mean())
                    if not info["finite"]:
                        problems.append(f"layer {li} {name}: non-finite weights")
                    if keep is not None:
                        info["pruned_nonzero"] = int((W[~keep] != 0).sum())
                        info["survivors_on_zero_code"] = int((W[keep] == 0).sum())
                        if info["pruned_nonzero"]:
                            problems.append(f"layer {li} {name}: {info['pruned_nonzero']} pruned positions do not decode to zero")
                rep["matrices"][f"{li}:{name}"] = info
    rep["ok"] = not problems
    if problems and strict:
        raise ValueError("container check failed:\n  " + "\n  ".join(problems))
    return rep


# ------------------------------------------------------------------ RAW artifacts
RAW_FIELDS = ("mask", "q", "scale", "zero", "col_scale")


def write_raw_artifact(path: str, layers: List[Dict[str, Dict[str, torch.Tensor]]], config: Optional[dict] = None,
                       stats: Optional[List[Dict[str, dict]]] = None) -> dict:
    """The compressor's output before packing, as the reference writes it
    (src/cobaltkernel/quantize_cobalt.py:439-443, :467): one `layer_XX.safetensors` per decoder
    layer holding `<name>.{mask,q,scale,zero,col_scale}` for every linear of the layer
    (src/cobaltkernel/pack_cobalt.py:3-11), and a `manifest.json` with the run's configuration
    and per-matrix entries (`shape`, `bits`, ...)."""
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    manifest = {"config": dict(config or {}), "layers": {}}
    for li, mats in enumerate(layers):
        tensors, entries = {}, {}
        for name, raw in mats.items():
            for f in RAW_FIELDS:
                tensors[f"{name}.{f}"] = raw[f].detach().cpu().contiguous()
            e = {"shape": [int(raw["q"].shape[0]), int(raw["q"].shape[1])]}
            if stats is not None:
                e.update(stats[li].get(name, {}))
            entries[name] = e
        save_file(tensors, os.path.join(path, f"layer_{li:02d}.safetensors"))
        manifest["layers"][str(li)] = entries
    with open(os.path.join(path, "manifest.json"), "w") as f:
        json.dump(manifest, f, indent=1)
    return manifest


def read_raw_artifact(path: str) -> Tuple[dict, List[Dict[str, Dict[str, torch.Tensor]]]]:
    """(manifest, layers[i][name] = {mask, q, scale, zero, col_scale}) of a RAW artifact directory;
    the manifest is {} if the directory has none."""
    from safetensors.torch import load_file
    manifest = {}
    mp = os.path.join(path, "manifest.json")
    if os.path.exists(mp):
        with open(mp) as f:
            manifest = json.load(f)
    files = sorted(n for n in os.listdir(path) if n.startswith("layer_") and n.endswith(".safetensors"))
    if not files:
        raise FileNotFoundError(f"no layer_XX.safetensors in {path}")
    layers = []
    for n in files:
        flat = load_file(os.path.join(path, n))
        mats: Dict[str, Dict[str, torch.Tensor]] = {}
        for key, t in flat.items():
            name, field = key.rsplit(".", 1)
            if field not in RAW_FIELDS:
                raise ValueError(f"{n}: unexpected tensor {key}")
            mats.setdefault(name, {})[field] = t
        for name, raw in mats.items():
            missing = [f for f in RAW_FIELDS if f not in raw]
            if missing:
                raise ValueError(f"{n}: {name} lacks {missing}")
        layers.append(mats)
    return manifest, layers


def raw_layout(raw: Dict[str, torch.Tensor], bits: Optional[int] = None) -> Tuple[int, int, int, Optional[int]]:
    """(layout, bits, group, keep) a RAW matrix packs to: dense if nothing is pruned, a blocked
    layout if every 32-column block keeps the same number of columns.  `bits` comes from the
    artifact's manifest when it has it, else from the largest code."""
    K, N = raw["q"].shape
    group = N // raw["scale"].shape[1]
    if bits is None:
        top = int(raw["q"].max())
        bits = 2 if top < 4 else 3 if top < 8 else 4 if top < 16 else 6 if top < 64 else 8
    keep_map = F.unpack_mask(raw["mask"], N)
    if bool(keep_map.all()):
        return (F.DENSE4 if (bits, group) == (4, 128) else F.DENSE8 if (bits, group) == (8, 128) else F.DENSEB), bits, group, None
    cnt = keep_map.reshape(K, N // F.BLOCK, F.BLOCK).sum(-1)
    k0 = int(cnt[0, 0])
    if bool((cnt == k0).all()):
        if (bits, group, k0) == (4, 128, 16):
            return F.BLK1632_4, 4, 128, 16
        if (bits, group, k0) == (6, 128, 16):
            return F.BLK1632_6, 6, 128, 16
        return F.BLKC, bits, group, k0
    raise ValueError("a mask without a fixed number of survivors per 32 columns packs to the variable-length "
                     "layouts, which this package reads but does not produce")

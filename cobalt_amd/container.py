"""CBK1 directories: `manifest.json` plus one `.bin` per decoder layer, each a concatenation of
256-byte aligned arrays that are, byte for byte, what the kernels read (reference:
docs/FORMAT.md:1-37 container, :126-151 fused matrices and `alias_of`; writer
src/cobaltkernel/pack_cobalt.py:390-505 and :561-714; loader src/cobaltkernel/runner.py:413-484).

The manifest is the reference's: `layers[i] = {file, matrices: {name: entry}, norms, bytes}`; an
entry holds K, N, G, layout, layout_name, arrays{data, row_off?, scale, zero, col_scale?: {off,
bytes}}, cs_rows, n_survivors, n_zero_fixed, stream_bytes, bpw.  A row-concatenated q|k|v matrix
carries `fused_from`, `row_ranges` and `cs_row_of`; the entries of its parts carry `alias_of` and
`alias_row_start`, byte ranges inside the fused arrays (their `data.bytes` has no 64-byte tail,
pack_cobalt.py:474-503) and a column scale of their own.  The layouts this package adds to the
reference's (BLKC, DENSEB) put their `bits`, `group` and `keep` into the entry.

Reading is offset-driven: a layer's blob is loaded once; the PackedMatrix of every matrix in it,
fused, alias or plain, is an offset table onto that one tensor.  On disk the rows are in the
reference's row-major order; `to_tiled()` reorders them for the decode kernel after the move to
the GPU.
"""
from __future__ import annotations

import json
import os
from collections import Counter
from typing import Dict, Iterator, List, Optional, Tuple

import numpy as np
import torch

from . import format as F

FORMAT_NAME = "CBK1"
FORMAT_VERSION = 1
QKV_PARTS = ("q_proj", "k_proj", "v_proj")
_ARRAYS = ("data", "row_off", "scale", "zero", "col_scale")


class _BlobWriter:
    """Appends arrays to one `.bin`, each on a 256-byte boundary (pack_cobalt.py:389-411)."""

    def __init__(self, path: str):
        self.f = open(path, "wb")
        self.pos = 0

    def _pad(self):
        pad = F._align(self.pos, F.ARR_ALIGN) - self.pos
        self.f.write(b"\0" * pad)
        self.pos += pad

    def put(self, t: torch.Tensor) -> dict:
        self._pad()
        raw = t.reshape(-1).clone(memory_format=torch.contiguous_format).view(torch.uint8).cpu().numpy().tobytes()
        off = self.pos
        self.f.write(raw)
        self.pos += len(raw)
        return {"off": off, "bytes": len(raw)}

    def close(self) -> int:
        self._pad()
        self.f.close()
        return self.pos


def _entry(pm: F.PackedMatrix, bw: _BlobWriter) -> dict:
    """Write the arrays of one matrix and return its manifest entry (pack_cobalt.py:414-434)."""
    e = {"K": pm.K, "N": pm.N, "G": pm.G, "layout": pm.layout, "layout_name": F.LAYOUT_NAME[pm.layout], "arrays": {}}
    for an in _ARRAYS:
        if an in pm.offs and (an != "col_scale" or pm.cs_rows):
            e["arrays"][an] = bw.put(pm.array(an))
    e.update(cs_rows=pm.cs_rows, n_survivors=pm.n_survivors, n_zero_fixed=pm.n_zero_fixed,
             stream_bytes=pm.stream_bytes(), bpw=pm.bpw())
    if pm.layout in (F.BLKC, F.DENSEB):
        e.update(bits=pm.bits, group=pm.group, keep=pm.keep)
    return e


def _alias_entry(fused: F.PackedMatrix, fe: dict, fused_name: str, k0: int, k1: int, cs_row: int, bw: _BlobWriter) -> dict:
    """Entry of rows [k0, k1) of a fused matrix: byte ranges inside the fused arrays, no bytes
    written but the part's own column scale (pack_cobalt.py:474-503)."""
    K, G = k1 - k0, fused.G
    stride = fused.data_bytes // fused.K
    fa = fe["arrays"]
    e = {"K": K, "N": fused.N, "G": G, "layout": fused.layout, "layout_name": F.LAYOUT_NAME[fused.layout],
         "arrays": {"data": {"off": fa["data"]["off"] + k0 * stride, "bytes": K * stride},
                    "scale": {"off": fa["scale"]["off"] + k0 * G * 2, "bytes": K * G * 2},
                    "zero": {"off": fa["zero"]["off"] + k0 * G, "bytes": K * G}}}
    e["arrays"]["col_scale"] = bw.put(fused.array("col_scale").view(fused.cs_rows, fused.N)[cs_row])
    share = (k1 - k0) / max(fused.K, 1)
    e.update(cs_rows=1, n_survivors=int(round(fused.n_survivors * share)), n_zero_fixed=0, alias_of=fused_name,
             alias_row_start=k0, stream_bytes=K * stride + K * G * 3)
    e["bpw"] = 8.0 * e["stream_bytes"] / (K * fused.N)
    if fused.layout in (F.BLKC, F.DENSEB):
        e.update(bits=fused.bits, group=fused.group, keep=fused.keep)
    return e


def write_container(path: str, layers: List[Dict[str, F.PackedMatrix]], config: Optional[dict] = None,
                    aliases: bool = True) -> dict:
    """Write `layers[i][name]` (row-major PackedMatrix objects) as layer_%02d.bin + manifest.json in
    the reference's schema (pack_cobalt.py:561-714) and return the manifest.  A matrix with three
    column-scale rows is a row-concatenated q|k|v: its entry names the row ranges and, with
    `aliases`, the layer also gets `alias_of` entries for the three parts."""
    os.makedirs(path, exist_ok=True)
    every = [pm for mats in layers for pm in mats.values()]
    lay = Counter(pm.layout for pm in every).most_common(1)[0][0] if every else F.BLK1632_4
    bits = Counter(pm.bits for pm in every).most_common(1)[0][0] if every else 4
    group = Counter(pm.group for pm in every).most_common(1)[0][0] if every else F.GROUP
    manifest = {"format": FORMAT_NAME, "version": FORMAT_VERSION, "group_size": group, "bits": bits,
                "layout": F.LAYOUT_NAME[lay], "embed_layout": None, "layout_override": {}, "bits_override": {},
                "mixed_layout": any((pm.layout, pm.bits) != (lay, bits) for pm in every),
                "fuse_gateup": any("gateup" in m for m in layers), "fuse_qkv": any("qkv" in m for m in layers),
                "raw_dir": None, "raw_config": dict(config or {}), "layers": [], "embed": None, "lm_head": None,
                "misc": None}
    tot_p = tot_b = 0
    for li, mats in enumerate(layers):
        rec = {"file": f"layer_{li:02d}.bin", "matrices": {}, "norms": {}}
        bw = _BlobWriter(os.path.join(path, rec["file"]))
        try:
            for name, pm in mats.items():
                if pm.tiled:
                    raise ValueError(f"{name}: write the row-major order; the tiled order is a load-time transform")
                e = _entry(pm, bw)
                rec["matrices"][name] = e
                tot_p += pm.K * pm.N
                tot_b += e["stream_bytes"]
                if pm.cs_rows == 3:
                    s0, s1 = pm.cs_splits
                    parts = tuple(pm.meta.get("fused_from", QKV_PARTS))
                    rr = {parts[0]: [0, s0], parts[1]: [s0, s0 + s1], parts[2]: [s0 + s1, pm.K]}
                    e.update(fused_from=list(parts), row_ranges=rr, cs_row_of={n: i for i, n in enumerate(parts)})
                    if aliases and not any(n in mats for n in parts):
                        for i, n in enumerate(parts):
                            if rr[n][1] > rr[n][0]:
                                rec["matrices"][n] = _alias_entry(pm, e, name, rr[n][0], rr[n][1], i, bw)
        finally:
            rec["bytes"] = bw.close()
        manifest["layers"].append(rec)
    manifest["bpw"] = {"params": tot_p, "packed_bytes": tot_b, "bpw_packed": 8.0 * tot_b / max(tot_p, 1)}
    with open(os.path.join(path, "manifest.json"), "w") as f:
        json.dump(manifest, f, indent=1)
    return manifest


def layer_records(manifest: dict) -> Iterator[Tuple[int, str, Dict[str, dict]]]:
    """(index, blob file name, {matrix name: entry}) for every layer of a manifest."""
    for li, rec in enumerate(manifest.get("layers", [])):
        if not isinstance(rec, dict) or "file" not in rec or "matrices" not in rec:
            raise ValueError(f"layer {li} of the manifest has no `file` / `matrices`: not a {FORMAT_NAME} layer record")
        yield li, rec["file"], rec["matrices"]


def _cs_splits(e: dict) -> Tuple[int, int]:
    """Row counts of the first two column-scale ranges of a q|k|v entry, from its `row_ranges` and
    `cs_row_of` (pack_cobalt.py:638-640): rows [0, s0) use column-scale row 0, [s0, s0+s1) row 1,
    the rest row 2."""
    if int(e.get("cs_rows", 0)) != 3:
        return (0, 0)
    rr, co = e.get("row_ranges"), e.get("cs_row_of")
    if not rr or not co:
        raise ValueError("an entry with three column-scale rows needs row_ranges and cs_row_of")
    order = sorted(rr, key=lambda n: co[n])
    r = [tuple(int(v) for v in rr[n]) for n in order]
    if len(r) != 3 or [co[n] for n in order] != [0, 1, 2] or r[0][0] != 0 or r[1][0] != r[0][1] or r[2][0] != r[1][1] \
            or r[2][1] != int(e["K"]):
        raise ValueError(f"row_ranges {rr} do not tile the rows 0..{e['K']} in column-scale order")
    return (r[0][1] - r[0][0], r[1][1] - r[1][0])


def matrix_from_entry(e: dict, blob: torch.Tensor) -> F.PackedMatrix:
    """PackedMatrix view of one manifest entry onto its (already loaded) blob.  The `data` array of
    an owning entry ends in the 64-byte tail; that of an `alias_of` entry is rows only."""
    layout = int(e["layout"])
    bits, group, keep = F.canon(layout, e.get("bits"), e.get("group"), e.get("keep"))
    a = e["arrays"]
    offs = {k: int(v["off"]) for k, v in a.items()}
    K, N = int(e["K"]), int(e["N"])
    data_bytes = int(a["data"]["bytes"]) - (0 if e.get("alias_of") else F.BLOB_TAIL)
    for an, want in (("scale", K * (N // group) * 2), ("zero", K * (N // group))):
        if int(a[an]["bytes"]) != want:
            raise ValueError(f"{an} holds {a[an]['bytes']} bytes, want {want} for {K}x{N} with groups of {group}")
    cs_rows = int(e.get("cs_rows", 0))
    if cs_rows and int(a["col_scale"]["bytes"]) != cs_rows * N * 2:
        raise ValueError(f"col_scale holds {a['col_scale']['bytes']} bytes, want {cs_rows} rows of {N} halves")
    pm = F.PackedMatrix(blob, offs, K, N, layout, bits, group, keep, cs_rows, _cs_splits(e), data_bytes,
                        int(e.get("n_survivors", 0)), int(e.get("n_zero_fixed", 0)))
    pm.validate(deep=blob.device.type == "cpu")
    pm.flags |= F.zero_flags(int(pm.array("zero").max()), bits)
    if e.get("fused_from"):
        pm.meta["fused_from"] = list(e["fused_from"])
    return pm


def read_container(path: str, device="cpu", include_aliases: bool = True) -> Tuple[dict, List[Dict[str, F.PackedMatrix]]]:
    """(manifest, layers) with every blob read once and placed on `device`."""
    with open(os.path.join(path, "manifest.json")) as f:
        manifest = json.load(f)
    if manifest.get("format") != FORMAT_NAME:
        raise ValueError(f"{path}: not a {FORMAT_NAME} directory")
    layers = []
    for li, fn, entries in layer_records(manifest):
        blob = torch.from_numpy(np.fromfile(os.path.join(path, fn), dtype=np.uint8)).to(device)
        mats = {}
        for name, e in entries.items():
            if e.get("alias_of") and not include_aliases:
                continue
            try:
                mats[name] = matrix_from_entry(e, blob)
            except (ValueError, KeyError) as err:
                raise ValueError(f"{path}: layer {li} {name}: {err}") from err
        layers.append(mats)
    return manifest, layers


def total_stream_bytes(manifest: dict) -> int:
    """Weight bytes one pass over the model streams; entries with `alias_of` are views into a
    fused matrix and are not counted twice (docs/FORMAT.md:146-151)."""
    return sum(int(e["stream_bytes"]) for _, _, entries in layer_records(manifest) for e in entries.values()
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
    owned: List[dict] = []
    try:
        records = list(layer_records(man))
    except ValueError as err:
        problems.append(str(err))
        records = []
    for li, bn, entries in records:
        bp = os.path.join(path, bn)
        if not os.path.exists(bp):
            problems.append(f"missing blob {bn}")
            continue
        sizes[bn] = os.path.getsize(bp)
        for name, e in entries.items():
            alias = bool(e.get("alias_of"))
            if alias and e["alias_of"] not in entries:
                problems.append(f"{bn}:{name} is an alias of {e['alias_of']}, which the layer does not hold")
            if not alias:
                owned.append(e)
            for an, a in e["arrays"].items():
                # an alias points into the fused arrays, on a row boundary rather than an array boundary
                if a["off"] % F.ARR_ALIGN and not (alias and an != "col_scale"):
                    problems.append(f"{bn}:{name}.{an} starts at {a['off']}, not on a {F.ARR_ALIGN}-byte boundary")
                if a["off"] + a["bytes"] > sizes[bn]:
                    problems.append(f"{bn}:{name}.{an} runs past the blob ({a['off']}+{a['bytes']} > {sizes[bn]})")
    rep["blob_bytes"] = sum(sizes.values())
    params = sum(e["K"] * e["N"] for e in owned)
    if params:
        rep["bpw"] = 8.0 * sum(e["stream_bytes"] for e in owned) / params
        want = sum(e["bpw"] * e["K"] * e["N"] for e in owned) / params
        if abs(rep["bpw"] - want) > 1e-6:
            problems.append(f"bytes per weight recompute to {rep['bpw']:.6f}, the entries say {want:.6f}")
    if not problems:
        on_gpu = torch.device(device).type == "cuda"
        try:
            _, mats_by_layer = read_container(path, device=device, include_aliases=False)
        except ValueError as err:
            problems.append(str(err))
            mats_by_layer = []
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

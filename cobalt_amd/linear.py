"""`CobaltLinear`: the nn.Module that stands where the reference installs its quantised linear
modules (benchmarks/benchmark_suite.py:1175-1217 `SparseQuantLinear`, sinq/sinqlinear.py:257-281,
sinq/cprlinear.py:366-387): `forward(x[..., in]) -> [..., out]` in `x.dtype`, `+ bias` if present.
Its weight is one CBK1 byte image; the forward is the HIP library, nothing else."""
from __future__ import annotations

from typing import Callable, Dict, Optional, Union

import torch
import torch.nn as nn

from . import format as F
from . import ops

_META_FIELDS = ("K", "N", "layout", "bits", "group", "keep", "cs_rows", "cs_split0", "cs_split1",
                "data_bytes", "off_data", "off_row_off", "off_scale", "off_zero", "off_col_scale",
                "n_survivors", "flags")


class CobaltLinear(nn.Module):
    def __init__(self, packed: F.PackedMatrix, bias: Optional[torch.Tensor] = None, meta: Optional[dict] = None):
        super().__init__()
        self.in_features, self.out_features = packed.N, packed.K
        self.register_buffer("blob", packed.blob)
        self.register_buffer("cbk_meta", self._meta_of(packed))
        self.bias = nn.Parameter(bias.detach().clone(), requires_grad=False) if bias is not None else None
        self.meta = dict(meta or {})
        self._backend = "hip"

    @staticmethod
    def _meta_of(packed: F.PackedMatrix) -> torch.Tensor:
        o = packed.offs
        return torch.tensor(
            [packed.K, packed.N, packed.layout, packed.bits, packed.group, packed.keep, packed.cs_rows,
             packed.cs_splits[0], packed.cs_splits[1], packed.data_bytes, o["data"], o.get("row_off", -1),
             o["scale"], o["zero"], o.get("col_scale", -1), packed.n_survivors, packed.flags], dtype=torch.int64)

    # ---- construction ------------------------------------------------------------------
    @staticmethod
    def _pack(mask, q, scale, zero, col_scale, layout, bits, group, keep, cs_splits=(0, 0), tiled=False) -> F.PackedMatrix:
        """RAW arrays on a GPU are packed there by the library's kernel, others by the torch packer."""
        if q.is_cuda:
            from . import ops
            return ops.pack_raw(mask, q, scale, zero, col_scale, layout, bits, group, keep, cs_splits=cs_splits, tiled=tiled)
        pm = F.pack_raw(mask, q, scale, zero, col_scale, layout, bits, group, keep, cs_splits=cs_splits)
        return pm.to_tiled() if tiled else pm

    @classmethod
    def from_raw(cls, mask, q, scale, zero, col_scale, bias=None, layout=F.BLK1632_4, bits=None, group=None,
                 keep=None, meta=None, cs_splits=(0, 0), tiled=False) -> "CobaltLinear":
        """From the RAW per-matrix schema `<name>.{mask,q,scale,zero,col_scale}`
        (src/cobaltkernel/pack_cobalt.py:3-11); `tiled` asks for the decode kernel's byte order
        at once instead of the reference's row-major order."""
        return cls(cls._pack(mask, q, scale, zero, col_scale, layout, bits, group, keep, cs_splits, tiled), bias, meta)

    @classmethod
    def from_linear(cls, linear: nn.Module, X_cal: Optional[torch.Tensor] = None, H: Optional[torch.Tensor] = None,
                    sparsity: float = 0.5, bits: int = 4, group: int = 128, beta: float = 0.5, mask_block: int = 32,
                    meta=None, raw_sink: Optional[dict] = None, raw_name: Optional[str] = None,
                    tiled: bool = False) -> "CobaltLinear":
        """Compress an `nn.Linear` with CoBALT and pack it (the role of `CPRLinear.from_linear`,
        sinq/cprlinear.py:128-171, with the pipeline of src/cobaltkernel/quantize_cobalt.py:424-443).
        Calibration comes as activations X_cal [tokens, in_features] or as H = X^T X; without
        either, H = I (magnitude pruning, no OBS signal).  The module lands on the linear's device.
        `raw_sink[raw_name]` receives the RAW arrays {mask, q, scale, zero, col_scale} on the CPU."""
        from . import compress as Cp
        W = linear.weight.data
        if H is None:
            H = Cp.hessian(X_cal.to(W.device)) if X_cal is not None else torch.eye(W.shape[1], device=W.device)
        raw = Cp.cobalt_compress(W, H.to(W.device), sparsity, bits, group, beta, mask_block)
        if raw_sink is not None:
            raw_sink[raw_name or "linear"] = {f: raw[f].detach().cpu() for f in ("mask", "q", "scale", "zero", "col_scale")}
        layout, keep = Cp.layout_for(sparsity, bits, group, mask_block)
        pm = cls._pack(raw["mask"], raw["q"], raw["scale"], raw["zero"], raw["col_scale"], layout, bits, group, keep,
                       tiled=tiled)
        bias = linear.bias.data if getattr(linear, "bias", None) is not None else None
        return cls(pm, bias, meta)

    @classmethod
    def from_state(cls, blob: torch.Tensor, cbk_meta: torch.Tensor, bias: Optional[torch.Tensor] = None) -> "CobaltLinear":
        """From the two buffers a saved module holds in a state dict (`<name>.blob`, `<name>.cbk_meta`)."""
        if blob.dtype != torch.uint8 or cbk_meta.numel() != len(_META_FIELDS):
            raise ValueError("not the buffers of a CobaltLinear")
        self = cls.__new__(cls)
        nn.Module.__init__(self)
        d = dict(zip(_META_FIELDS, [int(t) for t in cbk_meta.tolist()]))
        self.in_features, self.out_features = d["N"], d["K"]
        self.register_buffer("blob", blob)
        self.register_buffer("cbk_meta", cbk_meta.to("cpu", torch.int64).clone())
        self.bias = nn.Parameter(bias.detach().clone(), requires_grad=False) if bias is not None else None
        self.meta = {}
        self._backend = "hip"
        self.packed()                                                 # raises on an inconsistent description
        return self

    @classmethod
    def from_sparse_quant_linear(cls, m: nn.Module, layout: Optional[int] = None) -> "CobaltLinear":
        """From the reference's unpacked module: buffers W_q [K,N], scales/zeros [K,G,1], mask [K,N],
        scale2 [1,N] or [N], `bias`, meta{'nbits','group_size'} (benchmark_suite.py:1178-1198,
        built at src/nosink.py:1351-1354).  A mask with the same survivor count in every aligned
        32-column block goes to the bitmap layout, any other mask to the dense one."""
        W_q, mask = m.W_q, m.mask
        K, N = W_q.shape
        scales, zeros = m.scales, m.zeros
        if scales.dim() != 3:
            raise ValueError("per-row (ungrouped) quantisation has no CBK1 layout; use a group size of 64 or 128")
        G = scales.shape[1]
        group = N // G
        bits = int(m.meta.get("nbits", 4)) if isinstance(getattr(m, "meta", None), dict) else 4
        keepm = mask != 0
        cnt = keepm.reshape(K, N // 32, 32).sum(-1)
        c0 = int(cnt[0, 0])
        uniform = bool((cnt == c0).all()) and c0 >= 1
        if layout is None:
            if uniform and bits in (2, 3, 4):
                layout = F.BLK1632_4 if (bits, c0, group) == (4, 16, 128) else F.BLKC
            else:
                layout = F.DENSE4 if (bits, group) == (4, 128) else F.DENSEB
        bias = m.bias.data if getattr(m, "bias", None) is not None else None
        pm = cls._pack(F.pack_mask(keepm), torch.round(W_q.float()).to(torch.int32), scales.reshape(K, G),
                       zeros.reshape(K, G), m.scale2.reshape(-1, N), layout, bits, group, c0 if uniform else None)
        return cls(pm, bias, getattr(m, "meta", None))

    # ---- the packed view ----------------------------------------------------------------
    def packed(self) -> F.PackedMatrix:
        v = [int(t) for t in self.cbk_meta.tolist()]
        d = dict(zip(_META_FIELDS, v))
        offs = {"data": d["off_data"], "scale": d["off_scale"], "zero": d["off_zero"]}
        if d["off_row_off"] >= 0:
            offs["row_off"] = d["off_row_off"]
        if d["off_col_scale"] >= 0:
            offs["col_scale"] = d["off_col_scale"]
        return F.PackedMatrix(self.blob, offs, d["K"], d["N"], d["layout"], d["bits"], d["group"], d["keep"],
                              d["cs_rows"], (d["cs_split0"], d["cs_split1"]), d["data_bytes"], d["n_survivors"],
                              flags=d["flags"]).validate()

    def _apply(self, fn, recurse=True):
        out = super()._apply(fn, recurse)
        # the integer description stays on the host and is never cast
        self._buffers["cbk_meta"] = self.cbk_meta.to("cpu", torch.int64)
        if self.blob.dtype != torch.uint8:
            raise TypeError("the packed image is bytes; a dtype cast (.half()/.float()) cannot apply to it")
        self._pm_cache = None
        return out

    _pm_cache = None

    def _pm(self) -> F.PackedMatrix:
        if self._pm_cache is None or self._pm_cache.blob.data_ptr() != self.blob.data_ptr():
            self._pm_cache = self.packed()
        return self._pm_cache

    def to_device_order(self, repack_sparse: bool = False) -> "CobaltLinear":
        """Reorder the packed image, once, into the 16-row tile-interleaved byte order the decode
        kernel streams with fully coalesced loads (a permutation of the same bytes; fixed-stride
        layouts only, a no-op otherwise).  Call it after the module is on its GPU.
        A SPARSE4 matrix (rows of different lengths, no code offsets in the row) gets the table of
        group offsets of SPARSE4X (0.125 bits per weight more, the same mask and code bytes), with
        which the 16-row matrix-core stream kernel takes it.
        `repack_sparse`: a survivor-stream matrix (SPARSE4 / SPARSE4X / SPARSE4E) is re-packed as
        DENSE4 in tiled order instead, for the fixed-stride kernels (about twice the stream
        kernel's decode rate): every weight keeps its value, the image grows from about 3.2 to
        4.19 bits per weight."""
        pm = self._pm()
        if pm.tiled:
            return self
        if "row_off" in pm.offs:
            from . import ops
            if repack_sparse and pm.blob.is_cuda:
                t = ops.transcode(pm, F.DENSE4, tiled=True)
            elif pm.layout == F.SPARSE4:
                t = ops.with_group_offsets(pm)                    # the same codes as SPARSE4X: see there
            else:
                return self
        else:
            t = pm.to_tiled()
        self._buffers["blob"] = t.blob
        self._buffers["cbk_meta"] = self._meta_of(t)
        self._pm_cache = None
        return self

    # ---- forward --------------------------------------------------------------------------
    def set_forward_backend(self, backend: str):
        """Same switch as SINQLinear.set_forward_backend (sinq/sinqlinear.py:272-278); this module
        has one backend."""
        if backend != "hip":
            raise ValueError(f"Backend {backend} not supported")
        self._backend = backend

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.linear(self._pm(), x, self.bias)

    def forward_act(self, x: torch.Tensor, act: str) -> torch.Tensor:
        """For a gate/up matrix (rows 2i gate, 2i+1 up): act(gate(x)) * up(x), [.., out_features / 2]."""
        return ops.linear_act(self._pm(), x, act, self.bias)

    def dequantize(self, dtype=torch.float32) -> torch.Tensor:
        return ops.dequant(self._pm(), dtype)

    def extra_repr(self) -> str:
        p = self._pm()
        return (f"in_features={p.N}, out_features={p.K}, layout={F.LAYOUT_NAME[p.layout]}, bits={p.bits}, "
                f"group={p.group}, keep={p.keep}/32, bpw={p.bpw():.4f}, bias={self.bias is not None}")


def patch_model(model: nn.Module, replace: Union[Dict[str, nn.Module], Callable[[str, nn.Module], Optional[nn.Module]]]):
    """Install replacement modules by qualified name with `setattr(parent, leaf, new)`, the way the
    reference swaps its layers in (src/nosink.py:1353-1356, sinq/patch_model.py:585-609).
    `replace` is a {name: module} dict or a callback (name, module) -> module or None."""
    names = [n for n, _ in model.named_modules() if n]
    done = []
    for name in names:
        parent = model
        parts = name.split(".")
        try:
            for p in parts[:-1]:
                parent = getattr(parent, p)
            cur = getattr(parent, parts[-1])
        except AttributeError:
            continue
        new = replace.get(name) if isinstance(replace, dict) else replace(name, cur)
        if new is not None and new is not cur:
            setattr(parent, parts[-1], new)
            done.append(name)
    return done

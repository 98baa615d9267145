"""Whole-model installation: CoBALT-compress the seven linear layers of every decoder block of
a Hugging Face style causal LM and put `CobaltLinear` modules in their place.

What the reference does in two programs — calibrate and quantise layer by layer
(src/cobaltkernel/quantize_cobalt.py:361-443: one Hessian per group of linears that read the
same activation, taken from the *dense* model's activations unless `--seq-inputs` is given)
and swap modules in by name (sinq/patch_model.py:585-609, src/nosink.py:1353-1356) — is one
call here: `compress_model(model, calib_ids)`.

Everything runs on the device the model is on; the Hessians of `layers_per_pass` blocks are
held at a time (a Mistral-7B block needs 0.95 GB of float32 Hessians).
"""
from __future__ import annotations

from typing import Callable, Dict, Iterable, List, Optional, Sequence, Tuple

import torch
import torch.nn as nn

from . import format as F
from .linear import CobaltLinear

# names inside a decoder block (src/cobaltkernel/quantize_cobalt.py:30-38)
LINEARS = ("self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj", "self_attn.o_proj",
           "mlp.gate_proj", "mlp.up_proj", "mlp.down_proj")
# linears that read the same activation share one Hessian, hooked at the first of them
HGROUPS = {"attn_in": ("self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj"),
           "attn_out": ("self_attn.o_proj",),
           "mlp_in": ("mlp.gate_proj", "mlp.up_proj"),
           "mlp_out": ("mlp.down_proj",)}


def _sub(mod: nn.Module, path: str) -> Optional[nn.Module]:
    for p in path.split("."):
        mod = getattr(mod, p, None)
        if mod is None:
            return None
    return mod


def decoder_blocks(model: nn.Module) -> List[Tuple[str, nn.Module]]:
    """(qualified name, module) of every block that has all seven linears, in model order."""
    out = []
    for name, mod in model.named_modules():
        if all(isinstance(_sub(mod, l), (nn.Linear, CobaltLinear, FusedPart)) for l in LINEARS):
            out.append((name, mod))
    return out


def collect_hessians(model: nn.Module, blocks: Sequence[Tuple[str, nn.Module]],
                     calib_batches: Iterable[torch.Tensor],
                     forward: Optional[Callable[[nn.Module, torch.Tensor], object]] = None
                     ) -> Dict[Tuple[str, str], torch.Tensor]:
    """H = sum over all calibration tokens of x x^T (float32) for each (block, group), from one
    forward pass per batch through the model as it is."""
    Hs: Dict[Tuple[str, str], torch.Tensor] = {}
    hooks = []

    def mk(key):
        def hook(_mod, args):
            X = args[0].detach()
            X = X.reshape(-1, X.shape[-1]).float()
            if key not in Hs:
                Hs[key] = torch.zeros(X.shape[1], X.shape[1], dtype=torch.float32, device=X.device)
            Hs[key].addmm_(X.T, X)
        return hook

    for bname, blk in blocks:
        for g, names in HGROUPS.items():
            hooks.append(_sub(blk, names[0]).register_forward_pre_hook(mk((bname, g))))
    try:
        with torch.no_grad():
            for ids in calib_batches:
                if forward is not None:
                    forward(model, ids)
                else:
                    model(ids)
    finally:
        for h in hooks:
            h.remove()
    for key, H in Hs.items():
        if not bool(torch.isfinite(H).all()) or float(H.abs().amax()) == 0.0:
            raise RuntimeError(f"degenerate Hessian for {key}")       # quantize_cobalt.py:403-410
    return Hs


def compress_model(model: nn.Module, calib_ids: Optional[torch.Tensor] = None, sparsity: float = 0.5, bits: int = 4,
                   group: int = 128, beta: float = 0.5, mask_block: int = 32, layers_per_pass: int = 4,
                   batch_size: int = 4, device_order: bool = True,
                   bits_override: Optional[Dict[str, int]] = None,
                   sparsity_override: Optional[Dict[str, float]] = None, seq_inputs: bool = False,
                   fuse: bool = False,
                   forward: Optional[Callable[[nn.Module, torch.Tensor], object]] = None,
                   raw_out: Optional[str] = None) -> Dict[str, dict]:
    """Replace the linears of every decoder block by `CobaltLinear` modules compressed against
    the calibration tokens `calib_ids` [n, seq] (None: no calibration, H = I).  Per-matrix
    `bits_override` / `sparsity_override` are keyed by the names in LINEARS
    (quantize_cobalt.py:330-352).  The Hessians come from the dense model's activations: the new
    modules are installed when all blocks are done; with `seq_inputs` every pass of
    `layers_per_pass` blocks is installed at once and later passes calibrate on the compressed
    prefix (quantize_cobalt.py:444-452).  `fuse` row-fuses q|k|v and gate/up afterwards (fuse_model).
    `raw_out` also writes the RAW artifact of the run (one `layer_XX.safetensors` per block with
    `<name>.{mask,q,scale,zero,col_scale}` + manifest.json, quantize_cobalt.py:439-467), which
    `install_raw_artifact` and the reference's packer read.
    Returns {qualified linear name: {shape, layout, bpw,
    bits, sparsity}}."""
    blocks = decoder_blocks(model)
    if not blocks:
        raise ValueError("no decoder block with the linears " + ", ".join(LINEARS))
    bits_override = dict(bits_override or {})
    sparsity_override = dict(sparsity_override or {})
    for k in list(bits_override) + list(sparsity_override):
        if k not in LINEARS:
            raise ValueError(f"override name not in LINEARS: {k}")
    was_training = model.training
    model.eval()
    report: Dict[str, dict] = {}
    pending: List[Tuple[nn.Module, str, nn.Module]] = []
    raw_layers: List[Dict[str, Dict[str, torch.Tensor]]] = []
    raw_stats: List[Dict[str, dict]] = []

    def install():
        for parent, attr, new in pending:
            setattr(parent, attr, new)
        pending.clear()

    for c0 in range(0, len(blocks), max(1, layers_per_pass)):
        chunk = [b for b in blocks[c0:c0 + max(1, layers_per_pass)]
                 if any(isinstance(_sub(b[1], l), nn.Linear) for l in LINEARS)]
        if not chunk:
            continue
        Hs = {}
        if calib_ids is not None:
            batches = (calib_ids[i:i + batch_size] for i in range(0, calib_ids.shape[0], batch_size))
            Hs = collect_hessians(model, chunk, batches, forward)
        for bname, blk in chunk:
            raws: Dict[str, Dict[str, torch.Tensor]] = {}
            rstats: Dict[str, dict] = {}
            for g, names in HGROUPS.items():
                H = Hs.pop((bname, g), None)
                for lname in names:
                    lin = _sub(blk, lname)
                    if not isinstance(lin, nn.Linear):
                        continue
                    sp = sparsity_override.get(lname, sparsity)
                    nb = bits_override.get(lname, bits)
                    mb = 0 if sp == 0.0 else mask_block
                    new = CobaltLinear.from_linear(lin, H=H, sparsity=sp, bits=nb, group=group, beta=beta,
                                                   mask_block=mb, raw_sink=raws if raw_out else None,
                                                   raw_name=lname.rsplit(".", 1)[1],
                                                   tiled=device_order and lin.weight.is_cuda)
                    rstats[lname.rsplit(".", 1)[1]] = dict(bits=nb, sparsity_target=sp, mask_block=mb)
                    if device_order and new.blob.is_cuda:
                        new.to_device_order()
                    pending.append((_sub(blk, lname.rsplit(".", 1)[0]), lname.rsplit(".", 1)[1], new))
                    pm = new.packed()
                    report[f"{bname}.{lname}" if bname else lname] = dict(
                        shape=[pm.K, pm.N], layout=pm.layout, bpw=pm.bpw(), bits=nb, sparsity=sp)
                del H
            if raw_out:
                raw_layers.append({n.rsplit(".", 1)[1]: raws[n.rsplit(".", 1)[1]] for n in LINEARS if n.rsplit(".", 1)[1] in raws})
                raw_stats.append(rstats)
        if seq_inputs:
            install()
    install()
    if raw_out:
        from . import container
        container.write_raw_artifact(raw_out, raw_layers, stats=raw_stats,
                                     config=dict(sparsity=sparsity, bits=bits, group_size=group, beta=beta,
                                                 mask_block=mask_block))
    if fuse:
        fuse_model(model, device_order)
    if was_training:
        model.train()
    return report


class FusedRows(nn.Module):
    """One packed matrix for several linears that read the same activation (q|k|v concatenated,
    gate/up interleaved): one kernel launch instead of two or three, and a prefill GEMM that
    fills the chip where k and v alone are too small to.  The decoder block keeps calling its
    `q_proj`, `k_proj`, ... ; they are `FusedPart` views that run the fused matrix on the first
    call with a new activation tensor and hand out column slices of that result."""

    def __init__(self, fused: CobaltLinear, slices: Sequence[Tuple[int, int, int]]):
        super().__init__()
        self.fused = fused
        self.slices = [tuple(s) for s in slices]                     # (start, stop, step) along the output
        self._x = None
        self._xv = -1
        self._y = None
        self._served = 0

    def part(self, x: torch.Tensor, idx: int) -> torch.Tensor:
        if self._x is not x or self._xv != x._version:
            self._x, self._xv, self._served = x, x._version, 0
            self._y = self.fused(x)
        lo, hi, st = self.slices[idx]
        y = self._y[..., lo:hi:st]
        self._served += 1
        if self._served >= len(self.slices):                          # every part has been asked for: let go
            self._x = self._y = None
            self._xv = -1
        return y


class FusedPart(nn.Module):
    def __init__(self, owner: FusedRows, idx: int, in_features: int, out_features: int):
        super().__init__()
        self.__dict__["_owner"] = owner                               # not a submodule: the first part registers it
        self.idx, self.in_features, self.out_features = idx, in_features, out_features
        if idx == 0:
            self.rows = owner

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self._owner.part(x, self.idx)


def _fuse_group(blk: nn.Module, names: Sequence[str], interleave: bool, device_order: bool) -> bool:
    mods = [_sub(blk, n) for n in names]
    if not all(isinstance(m, CobaltLinear) for m in mods):
        return False
    pms = [m.packed().to_rowmajor() for m in mods]
    try:
        fused_pm = F.fuse_rows(pms, interleave=interleave)
    except ValueError:
        return False                                                  # e.g. per-matrix overrides: leave them apart
    bias = None
    if any(m.bias is not None for m in mods):
        bs = [m.bias.data if m.bias is not None else torch.zeros(m.out_features, device=m.blob.device, dtype=torch.float16)
              for m in mods]
        bias = torch.stack(bs, 1).reshape(-1) if interleave else torch.cat(bs)
    fused = CobaltLinear(fused_pm, bias)
    if device_order and fused.blob.is_cuda:
        fused.to_device_order()
    if interleave:
        slices = [(0, fused_pm.K, 2), (1, fused_pm.K, 2)]
    else:
        edges = [0]
        for p in pms:
            edges.append(edges[-1] + p.K)
        slices = [(edges[i], edges[i + 1], 1) for i in range(len(pms))]
    owner = FusedRows(fused, slices)
    for i, n in enumerate(names):
        setattr(_sub(blk, n.rsplit(".", 1)[0]), n.rsplit(".", 1)[1], FusedPart(owner, i, pms[i].N, pms[i].K))
    return True


def _gate_act_of(mlp: nn.Module) -> Optional[str]:
    """'gelu_tanh' or 'silu' if `mlp.act_fn` is that function (checked on values), else None."""
    fn = getattr(mlp, "act_fn", None)
    if not callable(fn):
        return None
    t = torch.linspace(-6.0, 6.0, 49)
    try:
        with torch.no_grad():
            v = fn(t)
    except Exception:
        return None
    if not isinstance(v, torch.Tensor) or v.shape != t.shape:
        return None
    if torch.allclose(v, torch.nn.functional.gelu(t, approximate="tanh"), atol=1e-6):
        return "gelu_tanh"
    if torch.allclose(v, torch.nn.functional.silu(t), atol=1e-6):
        return "silu"
    return None


def _gated_forward(self, x):
    """down(act(gate(x)) * up(x)) with the first half in one call on the fused gate/up matrix
    (EPI_GEGLU_BF16 / EPI_SWIGLU_BF16, src/cobaltkernel/csrc/cobalt_gemm.cuh:30-33)."""
    fused = self.gate_proj._owner.fused
    if isinstance(fused, CobaltLinear):
        h = fused.forward_act(x, self._cbk_act)
    else:                                                             # a dense twin of the fused matrix
        t = fused(x)
        g = t[..., 0::2]
        g = torch.nn.functional.gelu(g, approximate="tanh") if self._cbk_act == "gelu_tanh" else torch.nn.functional.silu(g)
        h = g * t[..., 1::2]
    return self.down_proj(h)


def _install_gated_forward(mlp: nn.Module) -> bool:
    """Give a gated MLP whose gate/up are fused (and whose forward is
    down_proj(act_fn(gate_proj(x)) * up_proj(x)), as the Hugging Face decoders' is) the one-call
    forward.  The module's own forward is run beside it once; it stays if the two disagree."""
    act = _gate_act_of(mlp)
    gp = getattr(mlp, "gate_proj", None)
    if act is None or not isinstance(gp, FusedPart) or not isinstance(gp._owner.fused, CobaltLinear):
        return False
    fused = gp._owner.fused
    if not fused.blob.is_cuda:
        return False
    import types
    x = torch.randn(3, fused.in_features, device=fused.blob.device, dtype=torch.float16, generator=None) * 0.5
    with torch.no_grad():
        a = mlp(x).float()
        mlp._cbk_act = act
        mlp.forward = types.MethodType(_gated_forward, mlp)
        b = mlp(x).float()
    if not bool(torch.isfinite(b).all()) or float((a - b).norm()) > 2e-2 * float(a.norm()) + 1e-6:
        del mlp.forward
        del mlp._cbk_act
        return False
    return True


def fuse_model(model: nn.Module, device_order: bool = True, gated_mlp: bool = True) -> int:
    """Fuse q|k|v and gate/up of every decoder block whose linears are row-major or device-order
    `CobaltLinear` modules with matching configurations.  With `gated_mlp`, an MLP of the form
    down(act(gate(x)) * up(x)) with a tanh-GELU or SiLU gate then computes act(gate) * up in the
    same call as the fused matrix.  Returns the number of fused groups."""
    n = 0
    for _bname, blk in decoder_blocks(model):
        for names, il in ((HGROUPS["attn_in"], False), (HGROUPS["mlp_in"], True)):
            mods = [_sub(blk, x) for x in names]
            if all(isinstance(m, CobaltLinear) for m in mods):
                for m in mods:                                       # fusing works on the row-major bytes
                    pm = m._pm()
                    if pm.tiled:
                        t = pm.to_rowmajor()
                        m._buffers["blob"] = t.blob
                        m._buffers["cbk_meta"] = m._meta_of(t)
                        m._pm_cache = None
                ok = _fuse_group(blk, names, il, device_order)
                n += 1 if ok else 0
                if ok and il and gated_mlp:
                    _install_gated_forward(_sub(blk, names[0].rsplit(".", 1)[0]))
    return n


def install_raw_artifact(model: nn.Module, path: str, device_order: bool = True, fuse: bool = False) -> Dict[str, dict]:
    """Install a RAW artifact directory (layer_XX.safetensors per decoder block, the reference
    compressor's output, src/cobaltkernel/quantize_cobalt.py:439-467) into `model`: every linear
    of every block is packed (pack_cobalt.py:98-199) and replaced by a `CobaltLinear` that keeps
    the linear's bias and lands on its device.  Returns the same report as `compress_model`."""
    from . import container
    manifest, layers = container.read_raw_artifact(path)
    blocks = decoder_blocks(model)
    if len(layers) != len(blocks):
        raise ValueError(f"the artifact has {len(layers)} layers, the model {len(blocks)} decoder blocks")
    report: Dict[str, dict] = {}
    for li, ((bname, blk), mats) in enumerate(zip(blocks, layers)):
        entries = manifest.get("layers", {}).get(str(li), {})
        for lname in LINEARS:
            short = lname.rsplit(".", 1)[1]
            if short not in mats:
                raise ValueError(f"layer {li}: no {short} in the artifact")
            raw = mats[short]
            lin = _sub(blk, lname)
            K, N = raw["q"].shape
            if (lin.out_features, lin.in_features) != (K, N):
                raise ValueError(f"layer {li} {short}: artifact {K}x{N}, model {lin.out_features}x{lin.in_features}")
            layout, nb, grp, keep = container.raw_layout(raw, entries.get(short, {}).get("bits"))
            dev = lin.weight.device if isinstance(lin, nn.Linear) else lin.blob.device
            t = {f: raw[f].to(dev) for f in container.RAW_FIELDS}
            bias = lin.bias.data if getattr(lin, "bias", None) is not None else None
            new = CobaltLinear.from_raw(t["mask"], t["q"], t["scale"], t["zero"], t["col_scale"], bias=bias,
                                        layout=layout, bits=nb, group=grp, keep=keep,
                                        tiled=device_order and dev.type == "cuda")
            if device_order and new.blob.is_cuda:
                new.to_device_order()
            setattr(_sub(blk, lname.rsplit(".", 1)[0]), short, new)
            pm = new.packed()
            report[f"{bname}.{lname}" if bname else lname] = dict(shape=[K, N], layout=pm.layout, bpw=pm.bpw(), bits=nb,
                                                                 sparsity=1.0 - pm.n_survivors / float(K * N))
    if fuse:
        fuse_model(model, device_order)
    return report


def load_compressed_state_dict(model: nn.Module, state_dict: Dict[str, torch.Tensor], strict: bool = True):
    """Load the state dict of a compressed model into a model that still has its dense linears.
    The module class is picked from the keys, the way the reference's loader does
    ('W_high_packed' -> CPRLinear, 'W_q' -> SINQLinear, sinq/patch_model.py:1129-1149): a name
    with `<name>.blob` and `<name>.cbk_meta` becomes a `CobaltLinear` built from those buffers, on
    the device of the module it replaces; everything else goes through `load_state_dict`."""
    names = [k[: -len(".cbk_meta")] for k in state_dict if k.endswith(".cbk_meta") and k[: -len(".cbk_meta")] + ".blob" in state_dict]
    modules = dict(model.named_modules())
    for name in names:
        old = modules.get(name)
        if old is None:
            if strict:
                raise KeyError(f"the state dict packs {name}, which the model does not have")
            continue
        if isinstance(old, CobaltLinear):
            continue                                                  # already packed: an ordinary buffer load
        dev = next((p.device for p in old.parameters()), torch.device("cpu"))
        bias = state_dict.get(name + ".bias")
        new = CobaltLinear.from_state(state_dict[name + ".blob"].to(dev), state_dict[name + ".cbk_meta"],
                                      None if bias is None else bias.to(dev))
        if isinstance(old, nn.Linear) and (old.in_features, old.out_features) != (new.in_features, new.out_features):
            raise ValueError(f"{name}: packed {new.out_features}x{new.in_features}, model {old.out_features}x{old.in_features}")
        parent = modules[name.rsplit(".", 1)[0]] if "." in name else model
        setattr(parent, name.rsplit(".", 1)[-1], new)
    return model.load_state_dict(state_dict, strict=strict)


def dense_twin(model: nn.Module, dtype: Optional[torch.dtype] = None) -> nn.Module:
    """The same model with every `CobaltLinear` turned back into an `nn.Linear` that holds the
    dequantised weight: what the packed model computes, through the dense library GEMM.  Modifies
    `model` in place and returns it (use it on a copy)."""
    for name, mod in list(model.named_modules()):
        for child_name, child in list(mod.named_children()):
            if isinstance(child, CobaltLinear):
                W = child.dequantize(torch.float32)
                lin = nn.Linear(child.in_features, child.out_features, bias=child.bias is not None,
                                device=W.device, dtype=dtype or torch.float16)
                lin.weight.data.copy_(W)
                if child.bias is not None:
                    lin.bias.data.copy_(child.bias.data)
                setattr(mod, child_name, lin)
    return model

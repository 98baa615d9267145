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
        if all(isinstance(_sub(mod, l), (nn.Linear, CobaltLinear)) for l in LINEARS):
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
                   forward: Optional[Callable[[nn.Module, torch.Tensor], object]] = None) -> Dict[str, dict]:
    """Replace the linears of every decoder block by `CobaltLinear` modules compressed against
    the calibration tokens `calib_ids` [n, seq] (None: no calibration, H = I).  Per-matrix
    `bits_override` / `sparsity_override` are keyed by the names in LINEARS
    (quantize_cobalt.py:330-352).  The Hessians come from the dense model's activations: the new
    modules are installed when all blocks are done; with `seq_inputs` every pass of
    `layers_per_pass` blocks is installed at once and later passes calibrate on the compressed
    prefix (quantize_cobalt.py:444-452).  Returns {qualified linear name: {shape, layout, bpw,
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
                                                   mask_block=mb)
                    if device_order and new.blob.is_cuda:
                        new.to_device_order()
                    pending.append((_sub(blk, lname.rsplit(".", 1)[0]), lname.rsplit(".", 1)[1], new))
                    pm = new.packed()
                    report[f"{bname}.{lname}" if bname else lname] = dict(
                        shape=[pm.K, pm.N], layout=pm.layout, bpw=pm.bpw(), bits=nb, sparsity=sp)
                del H
        if seq_inputs:
            install()
    install()
    if was_training:
        model.train()
    return report


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

"""Whole-model installer on the CPU: block discovery, Hessian collection and module replacement
(the packed modules themselves only run on the GPU)."""
import types

import pytest
import torch
import torch.nn as nn

from cobalt_amd import format as F
from cobalt_amd import model as Mo
from cobalt_amd.linear import CobaltLinear


class _Attn(nn.Module):
    def __init__(s, h, kv):
        super().__init__()
        s.q_proj, s.k_proj, s.v_proj, s.o_proj = nn.Linear(h, h, bias=False), nn.Linear(h, kv, bias=False), \
            nn.Linear(h, kv, bias=True), nn.Linear(h, h, bias=False)

    def forward(s, x):
        return s.o_proj(torch.tanh(s.q_proj(x)) * s.k_proj(x).mean(-1, keepdim=True) + s.v_proj(x).mean(-1, keepdim=True))


class _Mlp(nn.Module):
    def __init__(s, h, i):
        super().__init__()
        s.gate_proj, s.up_proj, s.down_proj = nn.Linear(h, i, bias=False), nn.Linear(h, i, bias=False), nn.Linear(i, h, bias=False)

    def forward(s, x):
        return s.down_proj(torch.nn.functional.silu(s.gate_proj(x)) * s.up_proj(x))


class _Block(nn.Module):
    def __init__(s, h, kv, i):
        super().__init__()
        s.self_attn, s.mlp = _Attn(h, kv), _Mlp(h, i)

    def forward(s, x):
        x = x + s.self_attn(x)
        return x + s.mlp(x)


class _Toy(nn.Module):
    def __init__(s, h=256, kv=128, i=384, layers=3, vocab=64):
        super().__init__()
        s.embed = nn.Embedding(vocab, h)
        s.layers = nn.ModuleList([_Block(h, kv, i) for _ in range(layers)])
        s.lm_head = nn.Linear(h, vocab, bias=False)

    def forward(s, ids):
        x = s.embed(ids)
        for l in s.layers:
            x = l(x)
        return s.lm_head(x)


def test_blocks_are_found_and_hessians_are_sums_of_outer_products():
    torch.manual_seed(0)
    m = _Toy()
    blocks = Mo.decoder_blocks(m)
    assert [n for n, _ in blocks] == ["layers.0", "layers.1", "layers.2"]
    ids = torch.randint(0, 64, (5, 7))
    Hs = Mo.collect_hessians(m, blocks[:2], [ids[:3], ids[3:]])
    assert set(Hs) == {(b, g) for b in ("layers.0", "layers.1") for g in Mo.HGROUPS}
    X0 = m.embed(ids).reshape(-1, 256).float()                    # what layers.0's q/k/v read
    assert torch.allclose(Hs[("layers.0", "attn_in")], X0.T @ X0, rtol=1e-5, atol=1e-4)
    # the down projection reads the gated activation: its Hessian is [inter, inter]
    assert Hs[("layers.1", "mlp_out")].shape == (384, 384)
    assert not m.layers[0].self_attn.q_proj._forward_pre_hooks      # hooks are gone


def test_compress_model_replaces_every_linear_and_honours_overrides():
    torch.manual_seed(1)
    m = _Toy(layers=2)
    ids = torch.randint(0, 64, (4, 16))
    rep = Mo.compress_model(m, ids, sparsity=0.5, bits=4, group=128, layers_per_pass=1,
                            bits_override={"mlp.down_proj": 3}, sparsity_override={"self_attn.o_proj": 0.0})
    assert len(rep) == 14
    for li in range(2):
        blk = m.layers[li]
        for name in Mo.LINEARS:
            mod = Mo._sub(blk, name)
            assert isinstance(mod, CobaltLinear), name
        assert rep[f"layers.{li}.mlp.gate_proj"]["layout"] == F.BLK1632_4
        assert abs(rep[f"layers.{li}.mlp.gate_proj"]["bpw"] - 3.1875) < 1e-9
        assert rep[f"layers.{li}.mlp.down_proj"]["layout"] == F.BLKC and rep[f"layers.{li}.mlp.down_proj"]["bits"] == 3
        assert rep[f"layers.{li}.self_attn.o_proj"]["layout"] == F.DENSE4
        assert blk.self_attn.v_proj.bias is not None and blk.self_attn.q_proj.bias is None
    assert isinstance(m.lm_head, nn.Linear)                        # only decoder blocks are touched
    assert Mo.compress_model(m, ids) == {}                         # nothing left to do
    with pytest.raises(ValueError):
        Mo.compress_model(_Toy(layers=1), ids, bits_override={"lm_head": 4})
    with pytest.raises(ValueError):
        Mo.compress_model(nn.Linear(8, 8), ids)


def test_packed_forward_fails_loudly_without_a_gpu():
    m = _Toy(layers=1)
    Mo.compress_model(m, None)
    if not torch.cuda.is_available():
        with pytest.raises(Exception):
            m(torch.randint(0, 64, (1, 4)))


def test_fuse_rows_layouts():
    """q|k|v concatenation and gate/up interleaving of packed matrices, checked on the bytes."""
    a, b, c = (F.synth_packed(K, 256, F.BLK1632_4, seed=i) for i, K in enumerate((32, 16, 16)))
    f = F.fuse_rows([a, b, c])
    st = F.row_stride(F.BLK1632_4, 256)
    assert (f.K, f.cs_rows, f.cs_splits) == (64, 3, (32, 16))
    assert torch.equal(f.array("data")[32 * st: 48 * st], b.array("data")[: 16 * st])
    assert torch.equal(f.array("scale").view(64, 2)[48:], c.array("scale").view(16, 2))
    assert torch.equal(f.array("col_scale").view(3, 256)[1], b.array("col_scale").view(256))
    g = F.fuse_rows([b, c], interleave=True)
    assert (g.K, g.cs_rows) == (32, 2)
    rows = g.array("data")[: 32 * st].view(32, st)
    assert torch.equal(rows[0::2], b.array("data")[: 16 * st].view(16, st))
    assert torch.equal(rows[1::2], c.array("data")[: 16 * st].view(16, st))
    assert torch.equal(g.array("zero").view(32, 2)[1::2], c.array("zero").view(16, 2))
    with pytest.raises(ValueError):
        F.fuse_rows([a, b], interleave=True)                       # unequal row counts
    with pytest.raises(ValueError):
        F.fuse_rows([a, F.synth_packed(16, 256, F.DENSE4, seed=3)])


def test_fuse_model_structure():
    m = _Toy(layers=2)
    Mo.compress_model(m, None, fuse=True)
    blk = m.layers[0]
    assert isinstance(blk.self_attn.q_proj, Mo.FusedPart) and isinstance(blk.mlp.up_proj, Mo.FusedPart)
    assert isinstance(blk.self_attn.o_proj, CobaltLinear)
    qkv = blk.self_attn.q_proj.rows.fused
    assert (qkv.out_features, qkv.packed().cs_rows, qkv.packed().cs_splits) == (512, 3, (256, 128))
    assert qkv.bias is not None and qkv.bias.shape == (512,)       # v_proj had a bias
    assert float(qkv.bias[:384].abs().max()) == 0.0
    gu = blk.mlp.gate_proj.rows.fused
    assert (gu.out_features, gu.packed().cs_rows) == (768, 2)
    keys = [k for k in m.state_dict() if k.startswith("layers.0.")]
    assert sum(k.endswith("blob") for k in keys) == 4              # one packed image per fused group
    assert len(Mo.decoder_blocks(m)) == 2


def test_raw_artifact_round_trip_installs_the_same_bytes(tmp_path):
    """compress_model(raw_out=...) writes the compressor's output in the reference's RAW schema
    (layer_XX.safetensors with <name>.{mask,q,scale,zero,col_scale}, pack_cobalt.py:3-11);
    installing that directory into a fresh model gives byte-identical packed modules, with the
    overrides (3-bit down, dense o) found again from the artifact alone."""
    from cobalt_amd import container as Ct
    torch.manual_seed(1)
    m = _Toy(layers=2)
    ids = torch.randint(0, 64, (4, 16))
    out = str(tmp_path / "raw")
    rep = Mo.compress_model(m, ids, sparsity=0.5, bits=4, group=128, layers_per_pass=1,
                            bits_override={"mlp.down_proj": 3}, sparsity_override={"self_attn.o_proj": 0.0},
                            raw_out=out)
    manifest, layers = Ct.read_raw_artifact(out)
    assert len(layers) == 2 and set(layers[0]) == {n.rsplit(".", 1)[1] for n in Mo.LINEARS}
    raw = layers[1]["gate_proj"]
    assert raw["mask"].dtype == torch.uint8 and raw["mask"].shape == (384, 256 // 8)
    assert raw["q"].dtype == torch.uint8 and raw["q"].shape == (384, 256)
    assert raw["scale"].dtype == torch.float16 and raw["zero"].dtype == torch.float16 and raw["scale"].shape == (384, 2)
    assert raw["col_scale"].dtype == torch.float16 and raw["col_scale"].shape == (256,)
    assert manifest["layers"]["0"]["down_proj"]["bits"] == 3 and manifest["layers"]["0"]["down_proj"]["shape"] == [256, 384]
    assert manifest["config"]["group_size"] == 128
    torch.manual_seed(1)
    m2 = _Toy(layers=2)
    rep2 = Mo.install_raw_artifact(m2, out)
    assert set(rep2) == set(rep)
    for k in rep:
        assert rep2[k]["layout"] == rep[k]["layout"] and rep2[k]["bits"] == rep[k]["bits"], k
        assert abs(rep2[k]["bpw"] - rep[k]["bpw"]) < 1e-12
    for li in range(2):
        for name in Mo.LINEARS:
            a, b = Mo._sub(m.layers[li], name), Mo._sub(m2.layers[li], name)
            assert isinstance(b, CobaltLinear) and torch.equal(a.blob, b.blob), (li, name)
            assert (a.bias is None) == (b.bias is None)
    # an artifact of another depth, or a mask no fixed-stride layout holds, is refused
    with pytest.raises(ValueError):
        Mo.install_raw_artifact(_Toy(layers=3), out)
    bad = {f: t.clone() for f, t in layers[0]["q_proj"].items()}
    bad["mask"][0, 0] ^= 1
    with pytest.raises(ValueError):
        Ct.raw_layout(bad)


def test_state_dict_of_a_compressed_model_loads_into_a_dense_one():
    """The loader picks `CobaltLinear` from the keys `<name>.blob` / `<name>.cbk_meta`
    (the reference picks its module classes the same way, sinq/patch_model.py:1129-1149)."""
    torch.manual_seed(2)
    m = _Toy(layers=2)
    Mo.compress_model(m, torch.randint(0, 64, (2, 16)), bits_override={"mlp.up_proj": 2})
    sd = {k: v.clone() for k, v in m.state_dict().items()}
    torch.manual_seed(3)
    m2 = _Toy(layers=2)                                              # dense, other weights
    res = Mo.load_compressed_state_dict(m2, sd)
    assert not res.missing_keys and not res.unexpected_keys
    for li in range(2):
        for name in Mo.LINEARS:
            a, b = Mo._sub(m.layers[li], name), Mo._sub(m2.layers[li], name)
            assert isinstance(b, CobaltLinear) and torch.equal(a.blob, b.blob) and torch.equal(a.cbk_meta, b.cbk_meta)
            assert (a.bias is None and b.bias is None) or torch.equal(a.bias, b.bias)
            assert b._pm().bits == a._pm().bits
    assert torch.equal(m2.embed.weight, m.embed.weight) and isinstance(m2.lm_head, nn.Linear)
    # a truncated blob is caught when the module is built, not at the first launch
    bad = dict(sd); bad["layers.0.mlp.up_proj.cbk_meta"] = sd["layers.0.mlp.up_proj.cbk_meta"][:5]
    with pytest.raises(ValueError):
        Mo.load_compressed_state_dict(_Toy(layers=2), bad)
    with pytest.raises(KeyError):
        Mo.load_compressed_state_dict(_Toy(layers=1), sd)


def test_six_bit_override_lands_in_the_reference_layout():
    """bits 6 at 16 of 32 kept and group 128 is BLK1632_6 (4.1875 bits per weight,
    docs/FORMAT.md:78-81), not the generic bit-stream layout; the RAW artifact finds it again."""
    from cobalt_amd import container as Ct
    torch.manual_seed(0)
    m = _Toy(layers=1)
    rep = Mo.compress_model(m, torch.randint(0, 64, (2, 16)), bits_override={"mlp.down_proj": 6})
    r = rep["layers.0.mlp.down_proj"]
    assert r["layout"] == F.BLK1632_6 and r["bits"] == 6 and abs(r["bpw"] - 4.1875) < 1e-9
    pm = m.layers[0].mlp.down_proj.packed()
    raw = dict(mask=pm.array("data")[: pm.K * (pm.N // 2)].view(pm.K, pm.N // 2)[:, : pm.N // 8].contiguous(),
               q=torch.full((pm.K, pm.N), 63, dtype=torch.uint8), scale=torch.ones(pm.K, pm.N // 128).half())
    assert Ct.raw_layout(raw) == (F.BLK1632_6, 6, 128, 16)

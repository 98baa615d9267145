"""Whole-model installation on a Hugging Face decoder (random-initialised tiny Mistral; there are
no checkpoints here): the packed model's logits against the same model with every packed layer
turned back into a dense layer of its dequantised weight."""
import copy

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _tiny_mistral():
    tr = pytest.importorskip("transformers")
    cfg = tr.MistralConfig(vocab_size=512, hidden_size=256, intermediate_size=512, num_hidden_layers=2,
                           num_attention_heads=4, num_key_value_heads=2, max_position_embeddings=512,
                           sliding_window=None, attn_implementation="eager")
    torch.manual_seed(0)
    return tr.MistralForCausalLM(cfg).to(DEV, torch.float16).eval()


def test_hf_decoder_is_compressed_in_place_and_matches_its_dense_twin():
    from cobalt_amd import model as Mo
    from cobalt_amd.linear import CobaltLinear
    m = _tiny_mistral()
    g = torch.Generator().manual_seed(1)
    calib = torch.randint(0, 512, (8, 64), generator=g).to(DEV)
    rep = Mo.compress_model(m, calib, sparsity=0.5, bits=4, group=128, layers_per_pass=1)
    assert len(rep) == 14 and all(abs(r["bpw"] - 3.1875) < 1e-9 for r in rep.values())
    assert sum(isinstance(x, CobaltLinear) for x in m.modules()) == 14
    assert all(x._pm().tiled for x in m.modules() if isinstance(x, CobaltLinear))
    twin = Mo.dense_twin(copy.deepcopy(m), torch.float16)
    assert not any(isinstance(x, CobaltLinear) for x in twin.modules())
    # prefill (M = 300 rows: the 256 x 256 kernel), a short prompt (M = 24: its 64-token tile)
    # and single-token steps (the decode kernel)
    for shape in ((1, 300), (2, 12), (1, 1), (3, 1)):
        ids = torch.randint(0, 512, shape, generator=g).to(DEV)
        with torch.no_grad():
            a = m(ids).logits.float()
            b = twin(ids).logits.float()
        err = float((a - b).norm() / b.norm())
        assert err < 5e-3, (shape, err)                             # fp16 activations through two blocks


def test_six_bit_and_three_bit_overrides_match_the_dense_twin():
    from cobalt_amd import format as F, model as Mo
    m = _tiny_mistral()
    g = torch.Generator().manual_seed(5)
    calib = torch.randint(0, 512, (4, 32), generator=g).to(DEV)
    rep = Mo.compress_model(m, calib, bits_override={"mlp.down_proj": 6, "self_attn.o_proj": 3})
    assert rep["model.layers.0.mlp.down_proj"]["layout"] == F.BLK1632_6
    twin = Mo.dense_twin(copy.deepcopy(m), torch.float16)
    for shape in ((1, 300), (1, 40), (2, 1)):
        ids = torch.randint(0, 512, shape, generator=g).to(DEV)
        with torch.no_grad():
            a, b = m(ids).logits.float(), twin(ids).logits.float()
        assert float((a - b).norm() / b.norm()) < 5e-3, shape


def test_compressed_model_state_dict_round_trip():
    from cobalt_amd import model as Mo
    m = _tiny_mistral()
    Mo.compress_model(m, None)
    sd = {k: v.clone() for k, v in m.state_dict().items()}
    m2 = _tiny_mistral()
    Mo.compress_model(m2, None, sparsity=0.5)                       # same module structure, other bytes
    for k in sd:
        if k.endswith("blob"):
            sd[k] = sd[k].clone()
    m2.load_state_dict(sd)
    ids = torch.randint(0, 512, (1, 5), generator=torch.Generator().manual_seed(2)).to(DEV)
    with torch.no_grad():
        assert torch.equal(m(ids).logits, m2(ids).logits)


def test_fused_qkv_and_gate_up_match_the_separate_modules():
    """`fuse=True`: q|k|v become one matrix with three col_scale vectors, gate/up one with two by
    row parity; the block still calls its seven projections, three launches fewer per block."""
    from cobalt_amd import model as Mo
    from cobalt_amd.linear import CobaltLinear
    m = _tiny_mistral()
    g = torch.Generator().manual_seed(1)
    calib = torch.randint(0, 512, (8, 64), generator=g).to(DEV)
    Mo.compress_model(m, calib)
    f = copy.deepcopy(m)
    assert Mo.fuse_model(f) == 4
    packed = [x for x in f.modules() if isinstance(x, CobaltLinear)]
    assert len(packed) == 2 * 4                                       # per block: qkv, o, gate/up, down
    assert sorted(x._pm().cs_rows for x in packed) == [1, 1, 1, 1, 2, 2, 3, 3]
    # the MLPs compute silu(gate) * up in the call of the fused matrix; without that they slice
    mlps = [blk.mlp for _n, blk in Mo.decoder_blocks(f)]
    assert all(getattr(x, "_cbk_act", None) == "silu" for x in mlps)
    f2 = copy.deepcopy(m)
    Mo.fuse_model(f2, gated_mlp=False)
    assert not any(hasattr(blk.mlp, "_cbk_act") for _n, blk in Mo.decoder_blocks(f2))
    h = torch.randn(2, 7, 256, generator=g).to(DEV, torch.float16)
    with torch.no_grad():
        ya, yb = mlps[0](h).float(), f2.model.layers[0].mlp(h).float()
    assert float((ya - yb).norm() / yb.norm()) < 2e-3
    twin = Mo.dense_twin(copy.deepcopy(f), torch.float16)
    for shape in ((1, 300), (2, 12), (1, 1), (2, 1)):
        ids = torch.randint(0, 512, shape, generator=g).to(DEV)
        with torch.no_grad():
            a, b, c = f(ids).logits.float(), m(ids).logits.float(), twin(ids).logits.float()
        assert float((a - c).norm() / c.norm()) < 5e-3, shape
        assert float((a - b).norm() / b.norm()) < 5e-3, shape
    # a second call with new contents in the same tensor object must not see the cached result
    ids = torch.randint(0, 512, (1, 4), generator=g).to(DEV)
    with torch.no_grad():
        y1 = f(ids).logits.clone()
        ids.copy_(torch.randint(0, 512, (1, 4), generator=g).to(DEV))
        y2 = f(ids).logits
        assert not torch.equal(y1, y2) and float((y2.float() - m(ids).logits.float()).norm()) < 5e-3 * float(y2.float().norm())


def test_raw_artifact_installs_on_the_gpu(tmp_path):
    """The RAW artifact written beside a compression run, installed into a second model on the GPU
    (fused at installation), gives the logits of the first."""
    from cobalt_amd import model as Mo
    m = _tiny_mistral()
    g = torch.Generator().manual_seed(3)
    calib = torch.randint(0, 512, (4, 32), generator=g).to(DEV)
    out = str(tmp_path / "raw")
    Mo.compress_model(m, calib, raw_out=out)
    m2 = _tiny_mistral()
    rep = Mo.install_raw_artifact(m2, out, fuse=True)
    assert len(rep) == 14 and all(abs(r["bpw"] - 3.1875) < 1e-9 for r in rep.values())
    for shape in ((1, 40), (2, 1)):
        ids = torch.randint(0, 512, shape, generator=g).to(DEV)
        with torch.no_grad():
            a, b = m(ids).logits.float(), m2(ids).logits.float()
        assert float((a - b).norm() / a.norm()) < 5e-3, shape


def test_check_container_on_the_gpu(tmp_path):
    """The numerical half of the container checker: blobs on the GPU, dequantised by the library;
    finite values, every pruned position exactly zero."""
    from cobalt_amd import container as Ct, format as F
    layers = [{"q_proj": F.synth_packed(64, 256, F.BLK1632_4, seed=1),
               "up_proj": F.synth_packed(48, 384, F.BLKC, 2, 64, 23, seed=2),
               "down_proj": F.synth_packed(32, 512, F.DENSE4, seed=3)}]
    Ct.write_container(str(tmp_path), layers)
    rep = Ct.check_container(str(tmp_path), device=DEV)
    assert rep["ok"]
    q = rep["matrices"]["0:q_proj"]
    assert q["finite"] and q["pruned_nonzero"] == 0 and q["zero_fraction"] >= 0.5
    assert rep["matrices"]["0:up_proj"]["block_survivors"] == [23, 23]
    assert "pruned_nonzero" not in rep["matrices"]["0:down_proj"] and rep["matrices"]["0:down_proj"]["finite"]


def test_directory_written_by_the_reference_loads_and_runs():
    """tests/golden/cbk1_dir was written by the reference's `pack_artifact` with fused qkv and
    gate/up (tests/golden/make_container_vectors.py); cbk1_dir_expect.npz holds the reference's own
    decode.  Loaded onto the GPU, every matrix (fused, alias, plain) dequantises bit for bit to
    that decode, and the fused matrices multiply like their parts, through the row-major bytes as
    read and through the tiled order."""
    import hashlib
    import os
    from cobalt_amd import container as Ct, ops
    gold = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    exp = np.load(os.path.join(gold, "cbk1_dir_expect.npz"))
    man, layers = Ct.read_container(os.path.join(gold, "cbk1_dir"), device=DEV)
    mats = layers[0]
    W = {}
    for name, pm in mats.items():
        W[name] = ops.dequant(pm, torch.float32)
        w = W[name].cpu().numpy() + np.float32(0.0)
        assert np.array_equal(w[exp[f"{name}.rows"]], exp[f"{name}.values"] + np.float32(0.0)), name
        assert hashlib.sha256(np.ascontiguousarray(w).tobytes()).hexdigest() == bytes(exp[f"{name}.sha256"]).decode(), name
        if "alias_of" not in man["layers"][0]["matrices"][name]:
            assert torch.equal(ops.dequant(pm.to_tiled(), torch.float32), W[name]), name
    g = torch.Generator(device=DEV).manual_seed(3)
    for M in (1, 3, 40):
        x = torch.randn(M, 256, device=DEV, generator=g).half()
        for fused in (mats["qkv"], mats["qkv"].to_tiled()):
            y = ops.linear(fused, x, out_dtype=torch.float32)
            parts = torch.cat([ops.linear(mats[n], x, out_dtype=torch.float32) for n in ("q_proj", "k_proj", "v_proj")], 1)
            ref = x.double() @ W["qkv"].double().T
            tol = 2e-5 if M < 8 else 2e-3
            assert float((y.double() - ref).abs().max() / ref.abs().max()) < tol
            assert float((parts.double() - ref).abs().max() / ref.abs().max()) < tol
        gu = ops.linear(mats["gateup"].to_tiled(), x, out_dtype=torch.float32).double()
        ref = x.double() @ W["gateup"].double().T
        assert float((gu - ref).abs().max() / ref.abs().max()) < (2e-5 if M < 8 else 2e-3)
    rep = Ct.check_container(os.path.join(gold, "cbk1_dir"), device=DEV)
    assert rep["ok"] and rep["matrices"]["0:gateup"]["pruned_nonzero"] == 0

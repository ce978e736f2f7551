"""CPU-side checks of the layered models' plumbing: configuration, layer order, slots, step tables, the checkpoint
reader, the library's exported surface, and the plain implementation's own consistency."""

import json
import re
import struct
import subprocess
from pathlib import Path

import pytest
import torch

REPO = Path(__file__).resolve().parent.parent


def _cfg():
    return {
        "architecture": "Bavesun", "vocab": 19, "width": 12, "norm": {"eps": 1e-6}, "embedding": {"scale": 2.5},
        "token_side": {"dim": 2}, "loop": {"start": 1, "stop": 3, "times": 3},
        "layers": [
            {"type": "retention", "mlp": {"kind": "dense", "ff": 10},
             "mixer": {"heads": 2, "dim": 4, "vdim": 6, "decay": [0.5, 0.75], "rot": {"dims": 2, "base": 100.0}}},
            {"type": "latent_attention", "mlp": {"kind": "moe", "expert": {"ff": 5}, "router": {"experts": 3, "top": 2}},
             "mixer": {"heads": 3, "dim": 2, "rot_dim": 4, "vdim": 2, "kv_rank": 6, "scale": 0.4,
                       "rot": {"dims": 4, "base": 50.0}}},
            {"type": "retention", "mlp": None,
             "mixer": {"heads": 1, "dim": 2, "vdim": 2, "decay": [1.0], "rot": {"dims": 2, "base": 7.0}}},
            {"type": "latent_attention", "mlp": None,
             "mixer": {"heads": 1, "dim": 2, "rot_dim": 2, "vdim": 4, "kv_rank": 4, "scale": 0.5,
                       "rot": {"dims": 2, "base": 50.0}}},
        ]}


def test_config_reads_every_size_and_the_layer_order():
    from lit_gpt.config import LayeredConfig

    c = LayeredConfig.from_dict(_cfg())
    assert (c.vocab, c.width, c.norm_eps, c.embedding_scale, c.side_dim) == (19, 12, 1e-6, 2.5, 2)
    assert c.layer_runs == [0, 1, 2, 1, 2, 1, 2, 3]
    m = c.layers[1].mixer
    assert (m.kind, m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank, m.scale) == ("latent_attention", 3, 2, 4, 2, 6, 0.4)
    assert c.layers[1].mlp.experts == 3 and c.layers[1].mlp.top == 2 and c.layers[1].mlp.ff == 5
    assert c.layers[0].mixer.decay == [0.5, 0.75] and c.layers[2].mlp is None
    f = c.layers[3].mixer.rot.inv_freq()
    assert f == [1.0]
    assert c.layers[1].mixer.rot.inv_freq() == pytest.approx([1.0, 50.0 ** -0.5])
    d = _cfg()
    del d["loop"], d["token_side"]
    c2 = LayeredConfig.from_dict(d)
    assert c2.layer_runs == [0, 1, 2, 3] and c2.side_dim == 0


def test_config_rejects_what_does_not_fit():
    from lit_gpt.config import LayeredConfig

    for change in (lambda d: d["loop"].update(stop=9), lambda d: d["layers"][0]["mixer"].update(decay=[0.5]),
                   lambda d: d["layers"][1]["mlp"]["router"].update(top=4),
                   lambda d: d["layers"][0].update(type="convolution"),
                   lambda d: d["layers"][0]["mixer"]["rot"].update(dims=6)):
        d = _cfg()
        change(d)
        with pytest.raises(ValueError):
            LayeredConfig.from_dict(d)


def test_registry_picks_the_class_by_config_json(tmp_path):
    from lit_gpt.config import LayeredConfig, load_config, model_class

    (tmp_path / "config.json").write_text(json.dumps(_cfg()))
    c = load_config(tmp_path)
    assert isinstance(c, LayeredConfig)
    assert model_class(c).__name__ == "LayeredGPT"
    (tmp_path / "config.json").write_text(json.dumps({"architecture": "Nonesuch"}))
    with pytest.raises(ValueError, match="not registered"):
        load_config(tmp_path)


def test_tensor_shapes_name_every_checkpoint_tensor():
    from lit_gpt.config import LayeredConfig
    from lit_gpt.layered import LayeredGPT

    shapes = LayeredGPT.tensor_shapes(LayeredConfig.from_dict(_cfg()))
    assert shapes["embed"] == (19, 12) and shapes["side.embed"] == (19, 8) and shapes["final.norm"] == (12,)
    assert shapes["l0.mix.q"] == (8, 12) and shapes["l0.mix.v"] == (12, 12) and shapes["l0.mix.o"] == (12, 12)
    assert shapes["l1.mix.q"] == (18, 12) and shapes["l1.mix.dkv"] == (10, 12) and shapes["l1.mix.uk"] == (6, 6)
    assert shapes["l1.mix.uv"] == (6, 6) and shapes["l1.mix.sink"] == (3,) and shapes["l1.mix.dkv.norm"] == (6,)
    assert shapes["l1.mlp.router"] == (3, 12) and shapes["l1.mlp.e2.down"] == (12, 5)
    assert shapes["l0.mlp.gate"] == (10, 12) and shapes["l3.side.proj"] == (12, 2)
    assert not any(k.startswith("l2.mlp") for k in shapes)


def test_slot_pool_hands_out_the_lowest_free_slot():
    from generate.batch import SlotPool

    p = SlotPool()
    assert [p.take() for _ in range(4)] == [0, 1, 2, 3]
    p.give(2)
    p.give(0)
    assert p.take() == 0 and p.take() == 2 and p.take() == 4
    with pytest.raises(ValueError):
        p.give(9)
    p.give(1)
    with pytest.raises(ValueError):
        p.give(1)


def test_step_table():
    from lit_gpt.mixers import StepBatch

    s = StepBatch.build([(3, 0, [5, 6, 7]), (0, 10, [1])], torch.device("cpu"))
    assert (s.T, s.B) == (4, 2)
    assert s.tokens.tolist() == [5, 6, 7, 1] and s.slot.tolist() == [3, 3, 3, 0] and s.pos.tolist() == [0, 1, 2, 10]
    assert s.seq_start.tolist() == [0, 3, 4] and s.seq_slot.tolist() == [3, 0] and s.seq_pos0.tolist() == [0, 10]
    assert s.tokens.dtype == torch.int32
    with pytest.raises(ValueError):
        StepBatch.build([(0, 0, [])], torch.device("cpu"))


def test_safetensors_reader(tmp_path):
    from lit_gpt.utils import read_safetensors

    a = torch.randn(3, 5).to(torch.bfloat16)
    b = torch.arange(7, dtype=torch.int32)
    blob = a.view(torch.uint8).numpy().tobytes() + b.view(torch.uint8).numpy().tobytes()
    header = {"a": {"dtype": "BF16", "shape": [3, 5], "data_offsets": [0, 30]},
              "b": {"dtype": "I32", "shape": [7], "data_offsets": [30, 58]}, "__metadata__": {"x": "y"}}
    hj = json.dumps(header).encode()
    path = tmp_path / "m.safetensors"
    path.write_bytes(struct.pack("<Q", len(hj)) + hj + blob)
    out = read_safetensors(path)
    assert set(out) == {"a", "b"} and torch.equal(out["a"], a) and torch.equal(out["b"], b)
    header["a"]["data_offsets"] = [0, 28]
    hj = json.dumps(header).encode()
    path.write_bytes(struct.pack("<Q", len(hj)) + hj + blob)
    with pytest.raises(ValueError):
        read_safetensors(path)


def test_library_exports_every_header_symbol():
    from lit_gpt import seq_ops

    text = re.sub(r"/\*.*?\*/", "", (REPO / "include" / "litgpt_seq.h").read_text(), flags=re.S)
    declared = sorted(set(re.findall(r"\b(lgs_[a-z0-9_]+)\s*\(", text)))
    assert declared == sorted(seq_ops.SIGNATURES)
    if not seq_ops.LIB_PATH.is_file():
        subprocess.run(["make", "-C", str(REPO / "lit-gpt_amd" / "csrc"), "-j8", "seq"], check=True)
    lib = seq_ops.load_library()
    assert lib.lgs_version() >= 1
    rc = lib.lgs_linear(None, 1, 0, None, 0, 0, None, 1, 0, 1, 1, 1, 1, 0, 0, None, None, 0, 0, None)
    assert rc != 0 and b"null" in lib.lgs_last_error_string()
    with pytest.raises(RuntimeError, match="GPU tensor"):
        seq_ops.rmsnorm(torch.zeros(2, 8), torch.ones(8), offset=0.0, eps=1e-5)


def test_oracle_is_causal_and_loops_share_weights():
    """The plain implementation itself: a later token never changes earlier logits, rotations keep lengths, and the
    routing weights of the chosen experts sum to one."""
    from lit_gpt.config import LayeredConfig
    from lit_gpt.layered import LayeredGPT
    from oracle import bavesun as ob

    cfg = _cfg()
    w = LayeredGPT.random_weights(LayeredConfig.from_dict(cfg), seed=1)
    toks = [3, 1, 4, 1, 5, 9, 2, 6]
    full = ob.forward(cfg, w, toks)
    assert torch.allclose(ob.forward(cfg, w, toks[:5]), full[:5], atol=1e-12)
    assert ob.layer_order(cfg) == [0, 1, 2, 1, 2, 1, 2, 3]
    x = torch.randn(8, dtype=torch.float64)
    for f in (ob.rope_half, ob.rope_interleaved):
        y = f(x, 17, 6, 100.0)
        assert torch.allclose(y.norm(), x.norm()) and torch.equal(y[6:], x[6:])
        assert torch.allclose(f(x, 0, 6, 100.0), x)
    assert ob.rope_half(torch.tensor([1.0, 0, 0, 0], dtype=torch.float64), 1, 4, 100.0)[2] == pytest.approx(
        torch.sin(torch.tensor(1.0, dtype=torch.float64)).item())
    assert ob.rope_interleaved(torch.tensor([1.0, 0, 0, 0], dtype=torch.float64), 1, 4, 100.0)[1] == pytest.approx(
        torch.sin(torch.tensor(1.0, dtype=torch.float64)).item())

"""Host side of the layer-list models, no GPU: the safetensors reader, the configuration reader's mapping onto layer descriptors, the ctypes
mirror of the descriptors against the C header, and the plain statement's own invariances."""
import ctypes as C
import json
import os
import subprocess

import numpy as np
import pytest

import seq_oracle
from powerserve_amd import hip, safetensors_io, seqmodel, synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
L = synth.seq_layer
CFG = synth.seq_config(24, 30, [L("delta", 20, heads=4, kv_heads=2, dim=6, vdim=10, conv=4), L("wkv", None, heads=3, dim=8),
                                L("latent_attention", 16, heads=2, dim=6, vdim=10, q_rank=7, kv_rank=9, rot_dim=4, rot={"base": 77.0, "dims": 4},
                                  mask={"size": 5}, scale=0.25)], taps=2, eps=1e-5, logit_scale=0.75)


def test_safetensors_round_trip_and_rounding(tmp_path):
    a = np.array([1.0, 1.00390625, 1.01171875, -3.0e-5, 65504.0, 0.0], dtype=np.float32)  # 1 + 2^-8 ties to even (down), 1 + 3 * 2^-8 ties up
    bits = safetensors_io.f32_to_bf16_bits(a)
    back = (bits.astype(np.uint32) << 16).view(np.float32)
    assert back[1] == 1.0 and back[2] == np.float32(1.015625) and back[0] == 1.0 and back[5] == 0.0
    t = {"w": np.arange(12, dtype=np.float32).reshape(3, 4), "idx": np.arange(5, dtype=np.int32)}
    p = str(tmp_path / "x.safetensors")
    safetensors_io.write(p, t)
    st = safetensors_io.SafeTensors(p)
    assert st.dtype("w") == "BF16" and st.dtype("idx") == "I32" and st.shape("w") == (3, 4)
    assert np.array_equal(st.f32("w"), t["w"]) and np.array_equal(st.raw("idx"), t["idx"])
    with pytest.raises(ValueError):
        st.bf16_bits("idx")


class FakeUp:
    def __init__(self):
        self.vecs, self.mats = [], []

    def vec(self, a):
        self.vecs.append(np.array(a))
        return len(self.vecs)

    def mat(self, bits):
        self.mats.append(np.array(bits))
        return 1000 + len(self.mats)


def test_configuration_maps_onto_layer_descriptors(tmp_path):
    t = synth.write_seq_model_dir(str(tmp_path), CFG, 1)
    cfg = seqmodel.read_config(str(tmp_path))
    up = FakeUp()
    layers, top = seqmodel.ARCHITECTURES[cfg["architecture"]](cfg, safetensors_io.SafeTensors(str(tmp_path / "model.safetensors")), up)
    assert (top["width"], top["vocab"], top["canon_taps"], top["norm_offset"]) == (24, 30, 2, 1.0)
    assert abs(top["norm_eps"] - 1e-5) < 1e-12 and top["logit_scale"] == 0.75
    d, w, a = layers
    assert (d.kind, d.heads, d.kv_heads, d.dim, d.vdim, d.conv_taps, d.ff_kind, d.ff) == (seqmodel.MIX_DELTA, 4, 2, 6, 10, 4, seqmodel.FF_DENSE_XIELU, 20)
    assert (w.kind, w.heads, w.dim, w.vdim, w.decay_rank, w.ff_kind) == (seqmodel.MIX_WKV, 3, 8, 8, 8, seqmodel.FF_NONE)
    assert (a.kind, a.q_rank, a.kv_rank, a.rot_dim, a.rot_dims, a.window) == (seqmodel.MIX_LATENT, 7, 9, 4, 4, 5)
    assert abs(a.rot_base - 77.0) < 1e-6 and abs(a.scale - 0.25) < 1e-9
    # the fused input projection of the delta mixer: rows q | k | v | g | b | a
    cat = up.mats[d.in_cat - 1001]
    assert cat.shape == (2 * 2 * 6 + 2 * 4 * 10 + 2 * 4, 24)
    want = np.concatenate([safetensors_io.f32_to_bf16_bits(t["l0.mix." + n]) for n in ("q", "k", "v", "g", "b", "a")])
    assert np.array_equal(cat, want)
    assert up.mats[a.ukv - 1001].shape == (2 * 6 + 2 * 10, 9) and up.mats[a.in_cat - 1001].shape == (7 + 9 + 4, 24)
    assert up.vecs[w.mu - 1].shape == (5, 24)


def test_unknown_names_are_refused(tmp_path):
    bad = dict(CFG, architecture="Somethingelse")
    synth.write_seq_model_dir(str(tmp_path), bad, 1, tensors=synth.seq_tensors(CFG, 1))
    with pytest.raises(seqmodel.ConfigError):
        seqmodel.read_config(str(tmp_path))
    bad = json.loads(json.dumps(CFG))
    bad["layers"][1]["type"] = "conveyor"
    with open(tmp_path / "config.json", "w") as f:
        json.dump(bad, f)
    with pytest.raises(seqmodel.ConfigError):
        seqmodel.ARCHITECTURES["Ranutar"](bad, safetensors_io.SafeTensors(str(tmp_path / "model.safetensors")), FakeUp())
    bad = json.loads(json.dumps(CFG))
    bad["canon"]["taps"] = 3  # the file's tensors have two taps
    with pytest.raises(seqmodel.ConfigError):
        seqmodel.ARCHITECTURES["Ranutar"](bad, safetensors_io.SafeTensors(str(tmp_path / "model.safetensors")), FakeUp())


def test_ctypes_descriptors_match_the_header(tmp_path):
    src = tmp_path / "sz.c"
    src.write_text('#include <stdio.h>\n#include <stddef.h>\n#include "ps_hip.h"\nint main(void){printf("%zu %zu %zu %zu %zu %zu\\n", sizeof(ps_seq_layer), '
                   'offsetof(ps_seq_layer, norm1), offsetof(ps_seq_layer, kvnorm), sizeof(ps_seq_desc), offsetof(ps_seq_desc, embed), offsetof(ps_seq_desc, layers));return 0;}\n')
    exe = str(tmp_path / "sz")
    subprocess.run(["gcc", "-I" + os.path.join(ROOT, "include"), str(src), "-o", exe], check=True)
    got = [int(x) for x in subprocess.run([exe], check=True, capture_output=True, text=True).stdout.split()]
    assert got == [C.sizeof(hip.SeqLayer), hip.SeqLayer.norm1.offset, hip.SeqLayer.kvnorm.offset, C.sizeof(hip.SeqDesc), hip.SeqDesc.embed.offset,
                   hip.SeqDesc.layers.offset]


def test_plain_statement_is_causal_and_windowed():
    """what a later token is does not change earlier logits; a token outside every window and with the recurrent layers cut out does not matter"""
    t = synth.seq_tensors(CFG, 2)
    rng = np.random.default_rng(0)
    a = rng.integers(0, 30, 20)
    b = a.copy()
    b[12] = (b[12] + 1) % 30
    la, lb = seq_oracle.run(CFG, t, a), seq_oracle.run(CFG, t, b)
    assert np.array_equal(la[:12], lb[:12]) and np.abs(la[12:] - lb[12:]).max() > 1e-3
    only = synth.seq_config(24, 30, [CFG["layers"][2]], taps=2)
    t2 = synth.seq_tensors(only, 2)
    la, lb = seq_oracle.run(only, t2, a), seq_oracle.run(only, t2, b)
    # window 5 and a 2-tap input filter in front of the mixer and of the feed-forward: token 12 reaches positions 12 .. 12 + 4 + 1 + 1
    assert np.abs(la[19:] - lb[19:]).max() < 1e-12 and np.abs(la[12:19] - lb[12:19]).max() > 1e-6


def test_the_small_library_exports_what_its_models_need():
    if not os.path.exists(hip.SEQ_LIB_PATH):
        pytest.skip("lib/libps_hip_seq.so not built")
    lib = C.CDLL(hip.SEQ_LIB_PATH)
    assert not [n for n in hip.SEQ_EXPORTS if not hasattr(lib, n)]

"""MLX safetensors ingestion (rmlx_amd/loader.py) against the reference loader's own tests
(crates/rmlx-nn/src/safetensors_loader.rs:653-1060) and, on the GPU, against the oracle."""
import json
import os

import numpy as np
import pytest

from oracle import model
from tests.helpers import assert_close, make_weight, make_x


def _loader():
    from rmlx_amd import loader
    return loader


# ---- name mapping and config parsing: the reference's known answers -----------------------------------

def test_hf_name_to_rmlx():
    hf = _loader().hf_name_to_rmlx
    assert hf("model.layers.0.self_attn.q_proj.weight") == "layers.0.attention.q_proj.weight"
    assert hf("model.layers.5.mlp.gate_proj.weight") == "layers.5.feed_forward.gate_proj.weight"
    assert hf("model.layers.5.mlp.down_proj.scales") == "layers.5.feed_forward.down_proj.scales"
    assert hf("model.layers.3.input_layernorm.weight") == "layers.3.attention_norm.weight"
    assert hf("model.layers.3.post_attention_layernorm.weight") == "layers.3.ffn_norm.weight"
    assert hf("model.embed_tokens.weight") == "embedding.weight"          # :701-707
    assert hf("lm_head.weight") == "lm_head.weight"                        # :709-711
    assert hf("layers.0.self_attn.q_proj.weight") == "layers.0.attention.q_proj.weight"  # :714-720


def test_parse_quantization_config(tmp_path):
    ld = _loader()
    p = tmp_path / "config.json"
    p.write_text('{"quantization": {"bits": 4, "group_size": 64}}')
    assert ld.parse_quantization_config(p) == ld.QuantizationConfig(4, 64)      # :727-736
    p.write_text('{"quantization": {"bits": 8, "group_size": 32}}')
    assert ld.parse_quantization_config(p) == ld.QuantizationConfig(8, 32)      # :739-748
    p.write_text('{"model_type": "qwen2"}')
    assert ld.parse_quantization_config(p) is None                              # :751-758
    p.write_text('{"quantization": {"bits": 3, "group_size": 64}}')
    with pytest.raises(ld.SafetensorsLoadError, match="bits must be 4 or 8, got 3"):   # :761-768
        ld.parse_quantization_config(p)
    p.write_text('{"quantization": {"bits": 4, "group_size": 16}}')
    with pytest.raises(ld.SafetensorsLoadError, match="group_size must be 32, 64, or 128, got 16"):  # :771-778
        ld.parse_quantization_config(p)
    p.write_text('{"quantization": {"group_size": 64}}')
    with pytest.raises(ld.SafetensorsLoadError, match="missing or invalid 'bits'"):
        ld.parse_quantization_config(p)
    p.write_text("{not json")
    with pytest.raises(ld.SafetensorsLoadError, match="Parse"):
        ld.parse_quantization_config(p)
    with pytest.raises(ld.SafetensorsLoadError, match="Io"):
        ld.parse_quantization_config(tmp_path / "missing.json")


def test_container_roundtrip_and_triplets(tmp_path):
    ld = _loader()
    rng = np.random.default_rng(0)
    words, s, b = make_weight(rng, 8, 64, 4)
    tensors = {"a.weight": ("U32", words), "a.scales": ("F16", s), "a.biases": ("F16", b),
               "norm.weight": ("F32", np.arange(6, dtype=np.float32).reshape(2, 3)),
               "b.weight": ("F16", np.ones((2, 2), np.float16)), "b.scales": ("F16", np.ones((2, 1), np.float16))}
    path = tmp_path / "m.safetensors"
    ld.write_safetensors(path, tensors)
    st = ld.SafetensorsFile(path)
    assert sorted(st.names()) == sorted(tensors)
    for name, (dtype, arr) in tensors.items():
        d, shape, got = st.tensor(name)
        assert d == dtype and shape == list(arr.shape) and np.array_equal(got, arr)
    # only complete triplets count (b has no biases)
    assert ld.find_triplets(st.names()) == {"a": ("a.weight", "a.scales", "a.biases")}
    with pytest.raises(ld.SafetensorsLoadError, match="TensorNotFound"):
        st.tensor("nope")
    # the third-party writer produces a file this parser reads identically
    try:
        from safetensors.numpy import save_file
    except Exception:
        save_file = None
    if save_file is not None:
        p2 = tmp_path / "m2.safetensors"
        save_file({k: v for k, (_, v) in tensors.items()}, str(p2))
        st2 = ld.SafetensorsFile(p2)
        for name, (dtype, arr) in tensors.items():
            d, shape, got = st2.tensor(name)
            assert d == dtype and np.array_equal(got, arr)


def test_container_rejects_malformed(tmp_path):
    ld = _loader()
    p = tmp_path / "bad.safetensors"
    p.write_bytes(b"\x01\x02")
    with pytest.raises(ld.SafetensorsLoadError, match="Parse"):
        ld.SafetensorsFile(p)
    p.write_bytes((10**12).to_bytes(8, "little") + b"{}")
    with pytest.raises(ld.SafetensorsLoadError, match="invalid header length"):
        ld.SafetensorsFile(p)
    hdr = json.dumps({"t": {"dtype": "F32", "shape": [4], "data_offsets": [0, 64]}}).encode()
    p.write_bytes(len(hdr).to_bytes(8, "little") + hdr + b"\0" * 16)
    with pytest.raises(ld.SafetensorsLoadError, match="outside the file"):
        ld.SafetensorsFile(p)
    hdr = json.dumps({"t": {"dtype": "I64", "shape": [2], "data_offsets": [0, 16]}}).encode()
    p.write_bytes(len(hdr).to_bytes(8, "little") + hdr + b"\0" * 16)
    with pytest.raises(ld.SafetensorsLoadError, match="UnsupportedDtype.*I64"):   # :874-884
        ld.SafetensorsFile(p).tensor("t")


def test_weight_map_basic():
    m = _loader().SafetensorsWeightMap()                                        # :898-909
    assert m.is_empty() and len(m) == 0 and m.num_quantized() == 0 and not m.contains("foo")
    with pytest.raises(_loader().SafetensorsLoadError, match="foo"):
        m.get("foo")


# ---- GPU: load and run -----------------------------------------------------------------------------------

@pytest.mark.gpu
def test_load_plain_and_f16(hip, tmp_path):
    ld = _loader()
    from rmlx_amd import runtime as rt
    path = tmp_path / "model.safetensors"
    ld.write_safetensors(path, {"test_weight": ("F32", np.array([[1, 2], [3, 4]], np.float32)),
                                "embed": ("F16", np.ones((2, 2), np.float16))})
    wmap = ld.load_safetensors_weights(path)                                     # :915-974
    assert len(wmap) == 2 and wmap.contains("test_weight") and wmap.num_quantized() == 0
    t = wmap.get("test_weight")
    assert t.shape == (2, 2) and t.dtype == rt.F32 and t.numpy().tolist() == [[1.0, 2.0], [3.0, 4.0]]
    assert wmap.get("embed").dtype == rt.F16


@pytest.mark.gpu
@pytest.mark.parametrize("bits,gs", [(4, 64), (8, 64), (4, 32)])
def test_load_quantized_checkpoint_and_forward(hip, tmp_path, bits, gs):
    ld = _loader()
    from rmlx_amd import runtime as rt
    rng = np.random.default_rng(bits * 100 + gs)
    layers = {"model.layers.0.self_attn.q_proj": (128, 512), "model.layers.0.mlp.down_proj": (64, 2048)}
    tensors, ref_w = {}, {}
    for prefix, (n, k) in layers.items():
        words, s, b = make_weight(rng, n, k, bits, gs)
        tensors[f"{prefix}.weight"], tensors[f"{prefix}.scales"], tensors[f"{prefix}.biases"] = \
            ("U32", words), ("F16", s), ("F16", b)
        ref_w[prefix] = (words, s, b, n, k)
    tensors["model.norm.weight"] = ("F16", np.ones(512, np.float16))
    (tmp_path / "config.json").write_text(json.dumps({"quantization": {"bits": bits, "group_size": gs}}))
    # two shards, like model-0000x-of-0000y.safetensors
    names = list(tensors)
    p1, p2 = tmp_path / "model-00001-of-00002.safetensors", tmp_path / "model-00002-of-00002.safetensors"
    ld.write_safetensors(p1, {k: tensors[k] for k in names[:3]})
    ld.write_safetensors(p2, {k: tensors[k] for k in names[3:]})
    qc = ld.parse_quantization_config(tmp_path / "config.json")
    wmap = ld.load_safetensors_sharded([p1, p2], qc)
    assert sorted(wmap.quantized_names()) == sorted(layers) and wmap.names() == ["model.norm.weight"]
    for prefix, (words, s, b, n, k) in ref_w.items():
        ql = wmap.get_quantized(prefix)
        assert (ql.out_features, ql.in_features, ql.group_size, ql.bits) == (n, k, gs, bits)
        for m in (1, 20):
            x = make_x(rng, m, k)
            ref = model.qmm(x.astype(np.float64), words, s, b, gs, bits)
            out = ql.forward(rt.DeviceBuffer.from_numpy(x)).numpy()
            assert_close(out, ref, f"{prefix} bits={bits} gs={gs} M={m}")
    # without a quantization config the triplet members stay plain tensors (load_plain, :388-412)
    plain = ld.load_safetensors_weights(p1)
    assert plain.num_quantized() == 0 and len(plain) == 3

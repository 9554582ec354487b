"""GGUF and AutoGPTQ-safetensors readers: container parsing on the CPU, loaded tensors through qmatmul on the GPU."""
import json
import os

import numpy as np
import pytest
import torch

import oracle as O
from conftest import synth
from gguf_writer import (T_ARR, T_BOOL, T_F32, T_I32, T_STR, T_U32, T_U64, write_gguf)
from mojo_amd import QuantizationEncoding as QE
from mojo_amd.weights import GGUFWeights, load_gptq_config, load_gptq_linear

GGML_F32, GGML_Q4_0, GGML_Q4_K, GGML_Q5_K, GGML_Q6_K, GGML_BF16 = 0, 2, 12, 13, 14, 30


def _model_file(tmp_path, alignment=None, version=3):
    w, _ = synth(31, 48, 512, 1)
    f32 = np.arange(24, dtype=np.float32).reshape(2, 3, 4)
    bf = (np.arange(10, dtype=np.uint16) * 257).reshape(2, 5)
    q4k, q6k, q40 = O.quantize(O.Q4_K, w), O.quantize(O.Q6_K, w), O.quantize(O.Q4_0, w[:, :96])
    q5k = O.quantize(O.Q5_K, w)
    meta = [("general.architecture", T_STR, "llama"), ("llama.block_count", T_U32, 32),
            ("llama.rope.freq_base", T_F32, 500000.0), ("general.file_type", T_U64, 15), ("flag", T_BOOL, True),
            ("tokenizer.ggml.tokens", T_ARR, (T_STR, ["<s>", "</s>", "hé"])),
            ("tokenizer.ggml.token_type", T_ARR, (T_I32, [1, 2, -3]))]
    tensors = [("norm.weight", [4, 3, 2], GGML_F32, f32.tobytes()),
               ("blk.0.attn_q.weight", [512, 48], GGML_Q4_K, q4k.tobytes()),
               ("output.weight", [512, 48], GGML_Q6_K, q6k.tobytes()),
               ("blk.0.ffn_up.weight", [96, 48], GGML_Q4_0, q40.tobytes()),
               ("rope.bf16", [5, 2], GGML_BF16, bf.tobytes()),
               ("blk.0.attn_v.weight", [512, 48], GGML_Q5_K, q5k.tobytes())]
    path = write_gguf(os.path.join(tmp_path, "m.gguf"), meta, tensors, version=version, alignment=alignment)
    return path, dict(w=w, f32=f32, bf=bf, q4k=q4k, q6k=q6k, q40=q40, q5k=q5k)


@pytest.mark.parametrize("alignment,version", [(None, 3), (64, 3), (32, 2)])
def test_gguf_metadata_and_tensor_views(tmp_path, alignment, version):
    path, ref = _model_file(tmp_path, alignment, version)
    g = GGUFWeights(path)
    assert g.version == version and g.alignment == (alignment or 32) and g.data_offset % g.alignment == 0
    assert g.metadata["general.architecture"] == "llama" and g.metadata["llama.block_count"] == 32
    assert g.metadata["llama.rope.freq_base"] == np.float32(500000.0) and g.metadata["flag"] is True
    assert g.metadata["tokenizer.ggml.tokens"] == ["<s>", "</s>", "hé"]
    assert g.metadata["tokenizer.ggml.token_type"].tolist() == [1, 2, -3]
    assert list(g) == ["norm.weight", "blk.0.attn_q.weight", "output.weight", "blk.0.ffn_up.weight", "rope.bf16",
                       "blk.0.attn_v.weight"]
    assert g.encoding("blk.0.attn_v.weight") is QE.Q5_K and g.tensors["blk.0.attn_v.weight"].nbytes == 48 * 2 * 176
    q = g.tensors["blk.0.attn_q.weight"]
    assert q.shape == (48, 512) and q.ggml_type == "Q4_K" and q.encoding is QE.Q4_K and q.nbytes == 48 * 2 * 144
    assert (q.offset - g.data_offset) % g.alignment == 0
    assert g.encoding("output.weight") is QE.Q6_K and g.encoding("blk.0.ffn_up.weight") is QE.Q4_0
    assert g.encoding("norm.weight") is None
    np.testing.assert_array_equal(g.raw("norm.weight"), ref["f32"])
    np.testing.assert_array_equal(g.raw("rope.bf16"), ref["bf"])
    for name, key in (("blk.0.attn_q.weight", "q4k"), ("output.weight", "q6k"), ("blk.0.ffn_up.weight", "q40"),
                      ("blk.0.attn_v.weight", "q5k")):
        raw = g.raw(name)
        assert raw.dtype == np.uint8 and raw.shape == ref[key].shape
        np.testing.assert_array_equal(raw, ref[key])
    # the bytes decode to the weights they were made from (oracle dequantiser)
    deq = O.dequantize(O.Q4_K, np.ascontiguousarray(g.raw("blk.0.attn_q.weight")), 512)
    assert np.abs(deq - ref["w"]).max() < 0.02


def test_gguf_rejects_malformed_files(tmp_path):
    path, _ = _model_file(tmp_path)
    data = open(path, "rb").read()

    def variant(name, blob):
        p = os.path.join(tmp_path, name)
        with open(p, "wb") as f:
            f.write(blob)
        return p

    with pytest.raises(ValueError, match="magic"):
        GGUFWeights(variant("magic.gguf", b"GGML" + data[4:]))
    with pytest.raises(ValueError, match="version"):
        GGUFWeights(variant("v1.gguf", data[:4] + (1).to_bytes(4, "little") + data[8:]))
    with pytest.raises(ValueError, match="truncated|past the end"):
        GGUFWeights(variant("short.gguf", data[:len(data) - 100]))
    with pytest.raises(ValueError, match="truncated"):
        GGUFWeights(variant("header.gguf", data[:60]))
    w, _ = synth(32, 4, 256, 1)
    q = O.quantize(O.Q4_K, w).tobytes()
    with pytest.raises(ValueError, match="not aligned"):
        GGUFWeights(write_gguf(os.path.join(tmp_path, "mis.gguf"), [], [("a", [256, 4], GGML_Q4_K, q),
                                                                        ("b", [256, 4], GGML_Q4_K, q)], misalign="b"))
    with pytest.raises(ValueError, match="unknown ggml type"):
        GGUFWeights(write_gguf(os.path.join(tmp_path, "type.gguf"), [], [("a", [256, 4], 99, q)]))
    with pytest.raises(ValueError, match="multiple of"):
        GGUFWeights(write_gguf(os.path.join(tmp_path, "row.gguf"), [], [("a", [100, 4], GGML_Q4_K, q)]))


def _gptq_checkpoint(tmp_path, with_g_idx=True):
    from safetensors.numpy import save_file

    w, a = synth(33, 64, 512, 3)
    qw, sc, qz, gi = O.quantize_gptq(w)
    tensors = {"model.layers.0.mlp.up_proj.qweight": qw, "model.layers.0.mlp.up_proj.scales": sc.view(np.float16),
               "model.layers.0.mlp.up_proj.qzeros": qz, "model.norm.weight": np.ones(4, np.float32)}
    if with_g_idx:
        tensors["model.layers.0.mlp.up_proj.g_idx"] = gi
    path = os.path.join(tmp_path, "model.safetensors")
    save_file(tensors, path)
    with open(os.path.join(tmp_path, "quantize_config.json"), "w") as f:
        json.dump({"bits": 4, "group_size": 128, "desc_act": False, "sym": True, "damp_percent": 0.01}, f)
    return path, (qw, sc, qz, gi), a


@pytest.mark.parametrize("with_g_idx", [True, False])
def test_gptq_safetensors_loader(tmp_path, with_g_idx):
    path, (qw, sc, qz, gi), _ = _gptq_checkpoint(tmp_path, with_g_idx)
    cfg = load_gptq_config(str(tmp_path))
    assert (cfg.bits, cfg.group_size, cfg.desc_act, cfg.sym, cfg.quant_method) == (4, 128, False, True, "gptq")
    got = load_gptq_linear(path, "model.layers.0.mlp.up_proj", device="cpu")
    np.testing.assert_array_equal(got[0].numpy(), qw)
    np.testing.assert_array_equal(got[1].view(torch.int16).numpy(), sc.view(np.int16))
    np.testing.assert_array_equal(got[2].numpy(), qz)
    np.testing.assert_array_equal(got[3].numpy(), gi)
    with pytest.raises(KeyError, match="lacks"):
        load_gptq_linear(path, "model.layers.1.mlp.up_proj", device="cpu")


@pytest.mark.gpu
def test_loaded_tensors_feed_qmatmul(tmp_path):
    from mojo_amd import qmatmul

    path, ref = _model_file(tmp_path)
    g = GGUFWeights(path)
    _, a = synth(34, 48, 512, 3)
    for name, enc in (("blk.0.attn_q.weight", O.Q4_K), ("output.weight", O.Q6_K)):
        want = O.matmul_f32(enc, a, np.ascontiguousarray(g.raw(name)))
        got = qmatmul(g.encoding(name), None, torch.from_numpy(a).to("cuda:0"), g.tensor(name)).cpu().numpy()
        assert O.isclose(got, want, 1e-3, 1e-4).all()
    gpath, (qw, sc, qz, gi), a2 = _gptq_checkpoint(tmp_path)
    want = O.matmul_gptq(a2, qw, sc, qz)
    got = qmatmul(QE.GPTQ, load_gptq_config(str(tmp_path)), torch.from_numpy(a2).to("cuda:0"),
                  *load_gptq_linear(gpath, "model.layers.0.mlp.up_proj")).cpu().numpy()
    assert O.isclose(got, want, 1e-3, 1e-4).all()

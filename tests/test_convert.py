"""AutoGPTQ safetensors -> `.bin` converter (restating export.py:25-122).  The input checkpoint is synthetic
(no model is fetched): AutoGPTQ-layout tensors in the Hugging Face Llama naming, fp16 where real checkpoints
hold fp16.  What pins the result: every projection of the written file, dequantised through the `.bin`
layout, equals the dequantisation of the ORIGINAL tensors in the AutoGPTQ formula (fp64, exact), the dense
tensors are the fp32 casts, and the oracle decodes the file to the logits of an independent fp64 decoder."""
import json
import os

import numpy as np
import pytest

from llama2_rs import checkpoint as ck
from llama2_rs import convert as cv
import tests.test_oracle_loop as tol

save_file = pytest.importorskip("safetensors.numpy").save_file


def _make_checkpoint(tmp_path, d, seed=0, shards=2):
    rng = np.random.default_rng(seed)
    t = {}
    f16 = lambda *s: rng.normal(0.0, 0.02, size=s).astype(np.float16)
    t["model.embed_tokens.weight"] = f16(d.vocab_size + 3, d.dim)      # 3 extra rows: max_vocab_size cuts them
    t["lm_head.weight"] = f16(d.vocab_size + 3, d.dim)
    t["model.norm.weight"] = (1.0 + f16(d.dim)).astype(np.float16)
    orig = {}
    for i in range(d.n_layers):
        p = f"model.layers.{i}."
        t[p + "input_layernorm.weight"] = (1.0 + f16(d.dim)).astype(np.float16)
        t[p + "post_attention_layernorm.weight"] = (1.0 + f16(d.dim)).astype(np.float16)
        for name, n_in, n_out in (("self_attn.q_proj", d.dim, d.dim), ("self_attn.k_proj", d.dim, d.kv_dim),
                                  ("self_attn.v_proj", d.dim, d.kv_dim), ("self_attn.o_proj", d.dim, d.dim),
                                  ("mlp.gate_proj", d.dim, d.hidden_dim), ("mlp.down_proj", d.hidden_dim, d.dim),
                                  ("mlp.up_proj", d.dim, d.hidden_dim)):
            qw, qz, sc, gidx = ck.synth_autogptq_linear(rng, n_in, n_out, d.group_size)
            sc = sc.astype(np.float16)
            t[p + name + ".qweight"], t[p + name + ".qzeros"] = qw, qz
            t[p + name + ".scales"], t[p + name + ".g_idx"] = sc, gidx
            orig[(name, i)] = ck.dequant_autogptq(qw, qz, sc.astype(np.float32), gidx)  # fp64 [IN][OUT]
    names = sorted(t)
    for s in range(shards):                                             # a sharded checkpoint, as large ones are
        part = {k: t[k] for k in names[s::shards]}
        save_file(part, str(tmp_path / f"model-{s + 1:05d}-of-{shards:05d}.safetensors"))
    (tmp_path / "config.json").write_text(json.dumps({
        "hidden_size": d.dim, "intermediate_size": d.hidden_dim, "num_hidden_layers": d.n_layers,
        "num_attention_heads": d.n_heads, "num_key_value_heads": d.n_kv_heads, "rms_norm_eps": 1e-6,
        "vocab_size": d.vocab_size + 3}))
    (tmp_path / "quantize_config.json").write_text(json.dumps({"bits": 4, "group_size": d.group_size,
                                                               "desc_act": True}))
    return t, orig


@pytest.mark.parametrize("dims", [
    ck.Dims(dim=256, hidden_dim=512, n_layers=2, n_heads=2, n_kv_heads=2, vocab_size=96, seq_len=64, group_size=64),
    ck.Dims(dim=512, hidden_dim=768, n_layers=1, n_heads=4, n_kv_heads=2, vocab_size=80, seq_len=32, group_size=128),
], ids=["mha_g64", "gqa_g128"])
def test_converted_file_decodes_to_the_original_weights(tmp_path, dims, oracle):
    t, orig = _make_checkpoint(tmp_path, dims)
    out = str(tmp_path / "m.bin")
    d = cv.convert(str(tmp_path), out, max_vocab_size=dims.vocab_size, max_seq_len=dims.seq_len, log=lambda s: None)
    assert d == dims
    assert os.path.getsize(out) == ck.checkpoint_bytes(dims)
    h = ck.read_header(out)
    assert (h["dim"], h["hidden_dim"], h["n_layers"], h["n_heads"], h["vocab_size"], h["seq_len"],
            h["shared_weight"]) == (dims.dim, dims.hidden_dim, dims.n_layers, dims.n_heads, dims.vocab_size,
                                    dims.seq_len, False)
    img = np.fromfile(out, dtype=np.uint8)[ck.HEADER_BYTES:]
    w = tol._split_image(img, dims)
    assert w["eps"] == np.float32(1e-6)
    np.testing.assert_array_equal(w["emb"], t["model.embed_tokens.weight"][:dims.vocab_size].astype(np.float64))
    np.testing.assert_array_equal(w["wcls"], t["lm_head.weight"][:dims.vocab_size].astype(np.float64))
    np.testing.assert_array_equal(w["rms_final"], t["model.norm.weight"].astype(np.float64))
    for key, name in (("wq", "self_attn.q_proj"), ("wk", "self_attn.k_proj"), ("wv", "self_attn.v_proj"),
                      ("wo", "self_attn.o_proj"), ("w1", "mlp.gate_proj"), ("w2", "mlp.down_proj"),
                      ("w3", "mlp.up_proj")):
        for i in range(dims.n_layers):
            np.testing.assert_array_equal(w[key][i], orig[(name, i)].T, err_msg=f"{name} layer {i}")
        np.testing.assert_array_equal(w["rms_att"][i], t[f"model.layers.{i}.input_layernorm.weight"].astype(np.float64))
        np.testing.assert_array_equal(w["rms_ffn"][i],
                                      t[f"model.layers.{i}.post_attention_layernorm.weight"].astype(np.float64))
    # the oracle reads the file as the reference would and agrees with a plain fp64 decoder on the original weights
    o = oracle.Model(img, dims)
    o.new_state()
    toks = [1, 7, 42, 5]
    for pos, tk in enumerate(toks):
        got = o.transformer([tk], [pos])
    want = tol._forward_fp64(w, dims, toks)
    assert np.max(np.abs(got - want)) < 2e-4 * max(1.0, float(np.max(np.abs(want))))
    o.close()


def test_converter_rejects_what_the_format_cannot_hold(tmp_path):
    dims = ck.Dims(dim=256, hidden_dim=512, n_layers=1, n_heads=2, n_kv_heads=2, vocab_size=40, seq_len=16,
                   group_size=64)
    _make_checkpoint(tmp_path, dims, shards=1)
    (tmp_path / "quantize_config.json").write_text(json.dumps({"bits": 8, "group_size": 64}))
    with pytest.raises(ValueError):
        cv.convert(str(tmp_path), str(tmp_path / "m.bin"), log=lambda s: None)
    (tmp_path / "quantize_config.json").write_text(json.dumps({"bits": 4, "group_size": 48}))
    with pytest.raises(ValueError):
        cv.convert(str(tmp_path), str(tmp_path / "m.bin"), log=lambda s: None)
    (tmp_path / "quantize_config.json").write_text(json.dumps({"bits": 4, "group_size": 128}))
    with pytest.raises(ValueError):   # shapes no longer fit the declared group size
        cv.convert(str(tmp_path), str(tmp_path / "m.bin"), log=lambda s: None)


@pytest.mark.gpu
def test_converted_file_through_the_hip_loader(tmp_path, oracle):
    """convert() -> l2_model_open -> transformer<1> on the GPU: the logits and the greedy tokens of the
    converted file equal the oracle's on the same file."""
    from llama2_rs import ops
    dims = ck.Dims(dim=512, hidden_dim=768, n_layers=2, n_heads=4, n_kv_heads=2, vocab_size=200, seq_len=48,
                   group_size=128)
    _make_checkpoint(tmp_path, dims, seed=3)
    out = str(tmp_path / "m.bin")
    assert cv.convert(str(tmp_path), out, max_vocab_size=dims.vocab_size, max_seq_len=dims.seq_len,
                      log=lambda s: None) == dims
    img = np.fromfile(out, dtype=np.uint8)[ck.HEADER_BYTES:]
    m = ops.Model(out, dims)
    o = oracle.Model(img, dims)
    o.new_state()
    for pos, tk in enumerate([1, 7, 42, 5, 199]):
        want = o.transformer([tk], [pos])
        got = m.forward([tk], [pos])
        scale = np.maximum(np.abs(want), np.sqrt(np.mean(want.astype(np.float64) ** 2)))
        assert np.max(np.abs(got - want) / scale) < 1e-4, pos
    prompt = np.array([3, 150, 9, 77, 12], np.int32)
    got, _ = m.generate_greedy(prompt, 30, use_prefill=True)
    np.testing.assert_array_equal(got, o.generate_greedy(prompt, 30, use_prefill=True))
    m.close()
    o.close()

"""Configuration, registry and weight loading (no GPU)."""
import json
import os

import numpy as np
import pytest
import torch

import helpers as H
from allpaca_amd.config import ConfigError, LlamaConfig, read_config_json
from allpaca_amd.models import ARCHITECTURES, DecoderModel, architecture_of, describe_model
from allpaca_amd.parts import rope
from allpaca_amd.weights import (SafetensorsError, SafetensorsFile, WeightsError, load_tensors, write_model_folder,
                                 write_safetensors)
import plain_llama as P


def test_config_reads_every_key_and_defaults():
    c = LlamaConfig.from_dict(H.TINY_B)
    assert (c.vocab_size, c.hidden_size, c.num_hidden_layers, c.num_attention_heads, c.num_key_value_heads,
            c.head_dim, c.intermediate_size) == (1000, 192, 3, 6, 2, 32, 512)
    assert c.rms_norm_eps == 1e-6 and c.rope_theta == 500000.0 and not c.tie_word_embeddings
    assert c.rope_scaling.factor == 8.0 and c.rope_scaling.original_max_position_embeddings == 64
    d = dict(H.TINY_A)
    for k in ("num_key_value_heads", "head_dim", "rms_norm_eps", "rope_theta", "rope_scaling", "tie_word_embeddings"):
        d.pop(k)
    c = LlamaConfig.from_dict(d)
    # kv heads default to heads, head_dim to hidden/heads (model.rs:7920-7921, 366-372), eps 1e-5, theta 1e4
    assert c.num_key_value_heads == 4 and c.head_dim == 16 and c.rms_norm_eps == 1e-5 and c.rope_theta == 10000.0
    assert c.rope_scaling is None and c.tie_word_embeddings is False


def test_config_takes_the_rope_parameters_table_and_a_file_without_a_position_limit():
    """Newer files carry theta and the scaling under `rope_parameters` (sidecar.rs:17-29); `max_position_embeddings`
    fixes no tensor's shape and the reference does not read it."""
    d = dict(H.TINY_B)
    scaling, theta = d.pop("rope_scaling"), d.pop("rope_theta")
    d["rope_parameters"] = dict(scaling, rope_theta=theta)
    assert LlamaConfig.from_dict(d) == LlamaConfig.from_dict(H.TINY_B)
    d = dict(H.TINY_A, rope_parameters=dict(rope_type="default", rope_theta=12345.0))
    d.pop("rope_theta")
    c = LlamaConfig.from_dict(d)
    assert c.rope_theta == 12345.0 and c.rope_scaling is None
    assert LlamaConfig.from_dict(dict(H.TINY_A, rope_scaling=dict(rope_type="default"))).rope_scaling is None
    assert LlamaConfig.from_dict(dict(H.TINY_B, rope_scaling=dict(H.TINY_B["rope_scaling"], rope_type=None, type="llama3"))
                                 ).rope_scaling.factor == 8.0
    d = dict(H.TINY_A)
    d.pop("max_position_embeddings")
    assert LlamaConfig.from_dict(d).max_position_embeddings == 2048


@pytest.mark.parametrize("key", ["hidden_size", "num_hidden_layers", "num_attention_heads", "intermediate_size",
                                 "vocab_size"])
def test_config_required_keys(key):
    d = dict(H.TINY_A)
    d.pop(key)
    with pytest.raises(ConfigError, match=key):
        LlamaConfig.from_dict(d)


def test_config_refusals():
    with pytest.raises(ConfigError, match="multiple"):
        LlamaConfig.from_dict(dict(H.TINY_A, num_key_value_heads=3))
    with pytest.raises(ConfigError, match="hidden_act"):
        LlamaConfig.from_dict(dict(H.TINY_A, hidden_act="gelu"))
    with pytest.raises(ConfigError, match="experts"):
        LlamaConfig.from_dict(dict(H.TINY_A, num_local_experts=8))
    with pytest.raises(ConfigError, match="rope_type"):
        LlamaConfig.from_dict(dict(H.TINY_A, rope_scaling=dict(rope_type="yarn", factor=2.0)))
    with pytest.raises(ConfigError, match="low_freq_factor"):
        LlamaConfig.from_dict(dict(H.TINY_A, rope_scaling=dict(rope_type="llama3", factor=2.0)))
    with pytest.raises(ConfigError, match="even"):
        LlamaConfig.from_dict(dict(H.TINY_A, head_dim=15))
    with pytest.raises(ConfigError, match="attention_bias"):
        LlamaConfig.from_dict(dict(H.TINY_A, attention_bias=True))


def test_registry_by_architecture_then_model_type():
    assert architecture_of({"architectures": ["LlamaForCausalLM"]}).name == "llama"
    assert architecture_of({"architectures": ["Other"], "model_type": "llama"}).name == "llama"
    with pytest.raises(ConfigError, match="known: .*LlamaForCausalLM"):
        architecture_of({"architectures": ["GPT2LMHeadModel"], "model_type": "gpt2"})
    with pytest.raises(ConfigError, match="names no architecture"):
        architecture_of({})


def test_spec_is_data_and_sizes_come_from_the_config():
    _, cfg, spec = describe_model(H.TINY_C)
    assert [e.block for e in spec.plan] == [0, 1] and all(e.cache_of is None for e in spec.plan)
    names = DecoderModel(spec).param_specs()
    assert names["model.layers.1.self_attn.q_proj.weight"].shape == (5 * 48, 120)
    assert names["model.layers.0.self_attn.k_proj.weight"].shape == (48, 120)
    assert names["model.layers.0.mlp.down_proj.weight"].shape == (120, 200)
    assert names["model.norm.weight"].store == "float32"
    assert "lm_head.weight" not in names and "lm_head.weight" in spec.forbidden  # tied
    _, _, spec_b = describe_model(H.TINY_B)
    assert DecoderModel(spec_b).param_specs()["lm_head.weight"].shape == (1000, 192)


def test_product_rope_table_matches_the_plain_one():
    for cfg in (H.TINY_A, H.TINY_B, H.TINY_C):
        d = cfg["head_dim"]
        got = rope.inverse_frequencies(d, cfg["rope_theta"], cfg["rope_scaling"])
        assert np.allclose(got, P.rope_inv_freq(d, cfg["rope_theta"], cfg["rope_scaling"]), rtol=1e-14)
    # Tiny B's table has frequencies in all three regions of the llama3 rule
    lam = 2 * np.pi / P.rope_inv_freq(32, 500000.0)
    assert (lam < 64 / 4).any() and (lam > 64).any() and ((lam >= 16) & (lam <= 64)).any()


def folder(tmp_path, cfg=H.TINY_A, dtype=torch.float32):
    path = str(tmp_path / "m")
    tensors = write_model_folder(path, cfg, 0, dtype)
    return path, tensors


def specs(cfg):
    _, _, spec = describe_model(cfg)
    return DecoderModel(spec).param_specs(), spec.forbidden


def rewrite(path, tensors):
    write_safetensors(os.path.join(path, "model.safetensors"), tensors)


def test_weights_roundtrip_and_storage_rule(tmp_path):
    path, tensors = folder(tmp_path, H.TINY_B, torch.bfloat16)
    want, forbidden = specs(H.TINY_B)
    got = load_tensors(path, want, torch.bfloat16, forbidden)
    assert got["model.layers.0.mlp.up_proj.weight"].dtype == torch.bfloat16       # kept in bfloat16
    assert got["model.norm.weight"].dtype == torch.float32                        # norm weights in 32-bit
    assert torch.equal(got["lm_head.weight"], tensors["lm_head.weight"])
    wide = load_tensors(path, want, torch.float32, forbidden)
    assert wide["lm_head.weight"].dtype == torch.float32
    assert torch.equal(wide["lm_head.weight"], tensors["lm_head.weight"].float())  # widened exactly
    # a matrix stored in 32-bit stays in 32-bit in a bfloat16 run; float16 is widened, never narrowed
    t2 = dict(tensors)
    t2["lm_head.weight"] = tensors["lm_head.weight"].float() + 1e-4
    t2["model.embed_tokens.weight"] = tensors["model.embed_tokens.weight"].to(torch.float16)
    rewrite(path, t2)
    got = load_tensors(path, want, torch.bfloat16, forbidden)
    assert got["lm_head.weight"].dtype == torch.float32 and torch.equal(got["lm_head.weight"], t2["lm_head.weight"])
    assert got["model.embed_tokens.weight"].dtype == torch.float32


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    path, tensors = folder(tmp_path)
    want, forbidden = specs(H.TINY_A)
    bad = dict(tensors)
    del bad["model.layers.1.mlp.up_proj.weight"]
    del bad["model.norm.weight"]
    bad["model.layers.0.self_attn.q_norm.weight"] = torch.ones(16)
    bad["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(32, 64)
    bad["lm_head.weight"] = torch.zeros(256, 64)     # tied model: must not be there
    rewrite(path, bad)
    with pytest.raises(WeightsError) as e:
        load_tensors(path, want, torch.float32, forbidden)
    err = e.value
    assert err.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.0.self_attn.q_norm.weight"]
    assert err.wrong_shape == [("model.layers.0.self_attn.k_proj.weight", (32, 64), (64, 64))]
    assert any("lm_head.weight" in m and "tie_word_embeddings" in m for m in err.other)
    msg = str(err)
    for piece in ("missing tensors (2)", "unexpected tensors (1)", "wrong shape", "[32, 64]", "[64, 64]"):
        assert piece in msg


def test_a_tied_head_stored_twice_and_a_frequency_buffer_are_passed_over(tmp_path):
    """Some writers store a tied matrix under both names and a table of rotation frequencies: a copy, bit for bit,
    of the embedding is no error, a head that differs is; names ending in `.rotary_emb.inv_freq` are no parameters."""
    from allpaca_amd.models import DecoderModel, describe_model
    path, tensors = folder(tmp_path)
    _, _, spec = describe_model(H.TINY_A)
    want = DecoderModel(spec).param_specs()
    more = dict(tensors)
    more["lm_head.weight"] = tensors["model.embed_tokens.weight"].clone()
    more["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.ones(8)
    rewrite(path, more)
    got = load_tensors(path, want, torch.float32, spec.forbidden, spec.copies, spec.ignored_suffixes)
    assert set(got) == set(want)
    more["lm_head.weight"][3, 5] += 1.0
    rewrite(path, more)
    with pytest.raises(WeightsError) as e:
        load_tensors(path, want, torch.float32, spec.forbidden, spec.copies, spec.ignored_suffixes)
    assert any("lm_head.weight" in m and "differs" in m for m in e.value.other) and not e.value.unexpected


def test_tensors_are_found_under_their_other_names(tmp_path):
    """The reference tries an ordered list of names for every tensor: GGUF-style, HF, without the `model.` prefix,
    a few older spellings (crates/allpaca-safetensors/src/names.rs:26-107); a missing tensor is reported with every
    name tried (catalog.rs:117-141)."""
    from allpaca_amd.models import DecoderModel, describe_model
    path, tensors = folder(tmp_path, H.TINY_B)
    _, _, spec = describe_model(H.TINY_B)
    want = DecoderModel(spec).param_specs()
    assert spec.aliases["model.layers.2.mlp.up_proj.weight"] == [
        "blk.2.ffn_up.weight", "model.layers.2.mlp.up_proj.weight", "layers.2.mlp.up_proj.weight",
        "model.layers.2.mlp.w3.weight"]
    # every tensor under another of its names, a different one from tensor to tensor
    renamed, used = {}, set()
    for i, (name, t) in enumerate(tensors.items()):
        names = spec.aliases[name]
        renamed[names[i % len(names)]] = t
        used.add(i % len(names))
    assert len(used) >= 3 and ("blk.0.attn_q.weight" in renamed or "token_embd.weight" in renamed)
    rewrite(path, renamed)
    got = load_tensors(path, want, torch.float32, spec.forbidden, spec.copies, spec.ignored_suffixes, spec.aliases)
    assert set(got) == set(want) and all(torch.equal(got[k], tensors[k]) for k in want)
    # without the list, the same file is a file of unexpected tensors
    with pytest.raises(WeightsError):
        load_tensors(path, want, torch.float32, spec.forbidden, spec.copies, spec.ignored_suffixes)
    # a missing tensor names every candidate; one present twice is an error; another tensor is still unexpected
    bad = dict(tensors)
    del bad["model.layers.1.self_attn.o_proj.weight"]
    bad["blk.0.attn_q.weight"] = tensors["model.layers.0.self_attn.q_proj.weight"]
    bad["blk.0.attn_q_norm.weight"] = torch.ones(32)
    rewrite(path, bad)
    with pytest.raises(WeightsError) as e:
        load_tensors(path, want, torch.float32, spec.forbidden, spec.copies, spec.ignored_suffixes, spec.aliases)
    assert e.value.missing == ["model.layers.1.self_attn.o_proj.weight (also tried: blk.1.attn_output.weight, "
                               "layers.1.self_attn.o_proj.weight)"]
    assert e.value.unexpected == ["blk.0.attn_q_norm.weight"]
    assert any("more than one of its names" in m and "blk.0.attn_q.weight" in m for m in e.value.other)
    # a tied model: the head under its GGUF-style name is as forbidden as under its own
    path_a = str(tmp_path / "a")
    ta = write_model_folder(path_a, H.TINY_A, 0, torch.float32)
    _, _, spec_a = describe_model(H.TINY_A)
    want_a = DecoderModel(spec_a).param_specs()
    ta = dict(ta)
    ta["output.weight"] = torch.zeros(256, 64)
    write_safetensors(os.path.join(path_a, "model.safetensors"), ta)
    with pytest.raises(WeightsError) as e:
        load_tensors(path_a, want_a, torch.float32, spec_a.forbidden, spec_a.copies, spec_a.ignored_suffixes, spec_a.aliases)
    assert any("output.weight" in m and "tie_word_embeddings" in m for m in e.value.other) and not e.value.unexpected


def test_untied_model_needs_its_head(tmp_path):
    path, tensors = folder(tmp_path, H.TINY_B)
    want, forbidden = specs(H.TINY_B)
    bad = dict(tensors)
    del bad["lm_head.weight"]
    rewrite(path, bad)
    with pytest.raises(WeightsError) as e:
        load_tensors(path, want, torch.float32, forbidden)
    assert e.value.missing == ["lm_head.weight"]


def test_container_errors(tmp_path):
    # crates/allpaca-safetensors/src/parser.rs:93-160: short file, header overrun, bad JSON, unsupported dtype
    p = tmp_path / "x.safetensors"
    p.write_bytes(b"\x01\x02")
    with pytest.raises(SafetensorsError, match="too short"):
        SafetensorsFile(str(p))
    p.write_bytes((1 << 40).to_bytes(8, "little") + b"{}")
    with pytest.raises(SafetensorsError, match="overruns"):
        SafetensorsFile(str(p))
    p.write_bytes((4).to_bytes(8, "little") + b"{{{{")
    with pytest.raises(SafetensorsError, match="JSON"):
        SafetensorsFile(str(p))
    hdr = json.dumps({"a": {"dtype": "F8_E4M3", "shape": [2], "data_offsets": [0, 2]}}).encode()
    p.write_bytes(len(hdr).to_bytes(8, "little") + hdr + b"\0\0")
    with pytest.raises(SafetensorsError, match="unsupported dtype"):
        SafetensorsFile(str(p))
    hdr = json.dumps({"a": {"dtype": "F32", "shape": [2], "data_offsets": [0, 4]}}).encode()
    p.write_bytes(len(hdr).to_bytes(8, "little") + hdr + b"\0\0\0\0")
    with pytest.raises(SafetensorsError, match="does not fit"):
        SafetensorsFile(str(p))
    with pytest.raises(SafetensorsError, match="no model.safetensors"):
        load_tensors(str(tmp_path / "nowhere"), {}, torch.float32)
    with pytest.raises(ConfigError, match="no config.json"):
        read_config_json(str(tmp_path))


def test_shards_and_duplicates(tmp_path):
    path, tensors = folder(tmp_path)
    want, forbidden = specs(H.TINY_A)
    names = list(tensors)
    a = {n: tensors[n] for n in names[: len(names) // 2]}
    b = {n: tensors[n] for n in names[len(names) // 2:]}
    os.remove(os.path.join(path, "model.safetensors"))
    write_safetensors(os.path.join(path, "model-00001-of-00002.safetensors"), a)
    write_safetensors(os.path.join(path, "model-00002-of-00002.safetensors"), b)
    with pytest.raises(SafetensorsError, match="several"):
        load_tensors(path, want, torch.float32, forbidden)
    wm = {n: "model-00001-of-00002.safetensors" for n in a}
    wm.update({n: "model-00002-of-00002.safetensors" for n in b})
    with open(os.path.join(path, "model.safetensors.index.json"), "w") as f:
        json.dump({"weight_map": wm}, f)
    got = load_tensors(path, want, torch.float32, forbidden)
    assert all(torch.equal(got[n], tensors[n]) for n in names)
    b[names[0]] = tensors[names[0]]
    write_safetensors(os.path.join(path, "model-00002-of-00002.safetensors"), b)
    with pytest.raises(WeightsError, match="appears in both"):
        load_tensors(path, want, torch.float32, forbidden)


def test_random_folder_is_reproducible_and_independent_of_other_tensors(tmp_path):
    a = write_model_folder(str(tmp_path / "a"), H.TINY_A, 5)
    b = write_model_folder(str(tmp_path / "b"), H.TINY_A, 5)
    c = write_model_folder(str(tmp_path / "c"), H.TINY_A, 6)
    more = write_model_folder(str(tmp_path / "d"), dict(H.TINY_A, num_hidden_layers=3), 5)
    n = "model.layers.1.mlp.gate_proj.weight"
    assert torch.equal(a[n], b[n]) and not torch.equal(a[n], c[n]) and torch.equal(a[n], more[n])
    assert abs(a[n].std().item() - 0.02) < 0.002 and torch.all(a["model.norm.weight"] == 1.0)
    cfg, w = P.read_model_folder(str(tmp_path / "a"))      # the plain reader reads what the writer wrote
    assert cfg["hidden_size"] == 64 and np.array_equal(w[n], a[n].double().numpy())


def test_random_weights_are_a_function_of_seed_name_and_element():
    """Every element is a hash of (seed, tensor name, index): the same whatever else is made, in any order, and, the
    arithmetic being integer up to one float32 multiplication, on any device (tests/test_generate_gpu.py holds the GPU
    against this).  A few elements against the formula written out with Python integers."""
    import numpy as np
    from allpaca_amd.parts import ParamSpec
    from allpaca_amd.weights.random_init import _tensor_seed, random_tensors, unit_normal
    M = (1 << 64) - 1

    def element(base, i):
        x = (i * 0xD6E8FEB86659FD93 + base + 0x9E3779B97F4A7C15) & M
        z = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & M
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M
        z ^= z >> 31
        total = (z & 0xFFFF) + ((z >> 16) & 0xFFFF) + ((z >> 32) & 0xFFFF) + (z >> 48)
        return np.float32(total - 131070) * np.float32((3.0 / (2 ** 32 - 1)) ** 0.5)

    specs = {"a.weight": ParamSpec((33, 7)), "b.weight": ParamSpec((5, 4)), "n.weight": ParamSpec((9,), store="float32")}
    t = random_tensors(specs, 11, torch.float32, std=0.5, norm_std=0.25)
    base = _tensor_seed(11, "a.weight")
    for i in (0, 1, 100, 230):
        assert float(t["a.weight"].flatten()[i]) == float(element(base, i) * np.float32(0.5))
    assert float(t["n.weight"][3]) == float(np.float32(1.0) + element(_tensor_seed(11, "n.weight"), 3) * np.float32(0.25))
    alone = random_tensors({"b.weight": specs["b.weight"]}, 11, torch.float32, std=0.5)
    assert torch.equal(alone["b.weight"], t["b.weight"])
    assert not torch.equal(random_tensors(specs, 12, torch.float32, std=0.5)["a.weight"], t["a.weight"])
    x = unit_normal(7, 400000, torch.device("cpu"))
    assert abs(float(x.mean())) < 0.01 and abs(float(x.std()) - 1.0) < 0.01 and float(x.abs().max()) < 3.5

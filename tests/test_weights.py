import json
import os

import pytest
import torch
from safetensors.torch import load_file, save_file

from jax_llm_examples_amd.config import get_architecture
from jax_llm_examples_amd.engine import load_model
from jax_llm_examples_amd.weights import SafetensorsFile, WeightsError, write_random_model
from tiny_configs import TINY, tiny_config_json, write_tiny


def test_random_folder_is_read_by_the_safetensors_package_and_by_ours(model_dirs):
    d = model_dirs["B"]
    theirs = load_file(os.path.join(d, "model.safetensors"))
    ours = SafetensorsFile(os.path.join(d, "model.safetensors"))
    assert set(theirs) == set(ours.names())
    assert all(k.startswith("language_model.") for k in theirs)  # the multimodal checkpoint's prefix
    for k, v in theirs.items():
        assert torch.equal(ours.tensor(k), v)
    gu = theirs["language_model.model.layers.1.feed_forward.experts.gate_up_proj"]
    assert gu.shape == (8, 96, 128)  # [E, D, 2F] as the checkpoint stores it
    assert theirs["language_model.model.layers.1.feed_forward.router.weight"].dtype == torch.float32
    assert (theirs["language_model.model.norm.weight"] == 1).all()
    assert abs(float(gu.std()) - 0.02) < 2e-3


def test_same_seed_same_values_and_tensors_do_not_depend_on_each_other(tmp_path):
    a = load_file(os.path.join(write_tiny("A", str(tmp_path / "a1")), "model.safetensors"))
    b = load_file(os.path.join(write_tiny("A", str(tmp_path / "a2")), "model.safetensors"))
    assert all(torch.equal(a[k], b[k]) for k in a)
    top = tiny_config_json("A")
    top["num_hidden_layers"], top["no_rope_layers"] = 2, [1, 0]
    arch = get_architecture("Llama4ForCausalLM")
    write_random_model(arch, arch.parse_config(top), str(tmp_path / "a3"), TINY["A"]["seed"], torch.float32)
    c = load_file(str(tmp_path / "a3" / "model.safetensors"))
    assert torch.equal(c["model.layers.1.self_attn.q_proj.weight"], a["model.layers.1.self_attn.q_proj.weight"])


def test_layouts_after_loading(model_dirs):
    d = model_dirs["A"]
    raw = load_file(os.path.join(d, "model.safetensors"))
    model = load_model(d, "float32", "cpu")
    p = model.named_parameters()
    hq, hk, dh = 4, 2, 16
    assert torch.equal(p["layers.2.mixer.wqkv"][: hq * dh], raw["model.layers.2.self_attn.q_proj.weight"])
    assert torch.equal(p["layers.2.mixer.wqkv"][hq * dh: (hq + hk) * dh], raw["model.layers.2.self_attn.k_proj.weight"])
    assert torch.equal(p["layers.2.mixer.wqkv"][(hq + hk) * dh:], raw["model.layers.2.self_attn.v_proj.weight"])
    gu = raw["model.layers.0.feed_forward.experts.gate_up_proj"]  # [E, D, 2F]
    assert torch.equal(p["layers.0.feed_forward.w_gate_up"], gu.transpose(1, 2))  # held [E, 2F, D]
    assert torch.equal(p["layers.0.feed_forward.w_gate_up"][1, :128], gu[1, :, :128].T)  # gate half first
    assert torch.equal(p["layers.0.feed_forward.w_down"], raw["model.layers.0.feed_forward.experts.down_proj"].transpose(1, 2))
    assert torch.equal(p["layers.0.feed_forward.shared_gate_up"][128:], raw["model.layers.0.feed_forward.shared_expert.up_proj.weight"])


def test_dtype_policy(model_dirs, model_dirs_bf16):
    m = load_model(model_dirs["A"], "bfloat16", "cpu")  # float32 file, bfloat16 run
    p = m.named_parameters()
    assert p["layers.0.mixer.wqkv"].dtype == torch.bfloat16 and p["embed.weight"].dtype == torch.bfloat16
    raw = load_file(os.path.join(model_dirs["A"], "model.safetensors"))
    # a tensor stored in 32-bit that is always held in 32-bit stays exactly as stored
    assert p["layers.0.feed_forward.router"].dtype == torch.float32
    assert torch.equal(p["layers.0.feed_forward.router"], raw["model.layers.0.feed_forward.router.weight"])
    assert p["layers.0.mixer_norm.weight"].dtype == torch.float32
    m2 = load_model(model_dirs_bf16["A"], "bfloat16", "cpu")  # bfloat16 file: kept in bfloat16, bit for bit
    raw2 = load_file(os.path.join(model_dirs_bf16["A"], "model.safetensors"))
    assert torch.equal(m2.named_parameters()["lm_head.weight"], raw2["lm_head.weight"])
    m3 = load_model(model_dirs_bf16["A"], "float32", "cpu")
    assert torch.equal(m3.named_parameters()["lm_head.weight"], raw2["lm_head.weight"].float())


def test_integer_tensors_become_int32(tmp_path):
    from jax_llm_examples_amd.weights.bindings import TensorBinding
    from jax_llm_examples_amd.weights.loader import place

    target = torch.zeros(4, dtype=torch.int32)
    place(target, TensorBinding("t", (4,), "x"), torch.tensor([1, 2, 3, 4], dtype=torch.int64))
    assert target.dtype == torch.int32 and target.tolist() == [1, 2, 3, 4]


def test_one_error_lists_missing_unexpected_and_wrong_shapes(model_dirs, tmp_path):
    raw = load_file(os.path.join(model_dirs["A"], "model.safetensors"))
    del raw["model.layers.1.self_attn.o_proj.weight"], raw["model.norm.weight"]
    raw["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    raw["lm_head.weight"] = raw["lm_head.weight"][:, :32].contiguous()
    raw["vision_model.patch_embedding.weight"] = torch.zeros(3)  # ignored, not unexpected
    os.makedirs(tmp_path / "bad")
    save_file(raw, str(tmp_path / "bad" / "model.safetensors"))
    with open(tmp_path / "bad" / "config.json", "w") as f:
        json.dump(tiny_config_json("A"), f)
    with pytest.raises(WeightsError) as ei:
        load_model(str(tmp_path / "bad"), "float32", "cpu")
    e = ei.value
    assert sorted(e.missing) == ["model.layers.1.self_attn.o_proj.weight", "model.norm.weight"]
    assert e.unexpected == ["model.layers.0.self_attn.rotary_emb.inv_freq"]
    assert e.wrong_shape == [("lm_head.weight", (512, 32), (512, 64))]
    msg = str(e)
    assert "missing (2)" in msg and "unexpected (1)" in msg and "lm_head.weight is [512, 32], expected [512, 64]" in msg


def test_sharded_checkpoint_with_index(model_dirs, tmp_path):
    raw = load_file(os.path.join(model_dirs["A"], "model.safetensors"))
    names = sorted(raw)
    half = len(names) // 2
    os.makedirs(tmp_path / "sh")
    wm = {}
    for i, part in enumerate((names[:half], names[half:])):
        fn = f"model-0000{i + 1}-of-00002.safetensors"
        save_file({k: raw[k] for k in part}, str(tmp_path / "sh" / fn))
        wm.update({k: fn for k in part})
    with open(tmp_path / "sh" / "model.safetensors.index.json", "w") as f:
        json.dump({"weight_map": wm}, f)
    with open(tmp_path / "sh" / "config.json", "w") as f:
        json.dump(tiny_config_json("A"), f)
    a = load_model(str(tmp_path / "sh"), "float32", "cpu").named_parameters()
    b = load_model(model_dirs["A"], "float32", "cpu").named_parameters()
    assert all(torch.equal(a[k], b[k]) for k in b)


def _folder_with(tmp_path, name, files, index=None):
    d = tmp_path / name
    os.makedirs(d)
    for fn, tensors in files.items():
        save_file(tensors, str(d / fn))
    if index is not None:
        with open(d / "model.safetensors.index.json", "w") as f:
            json.dump({"weight_map": index}, f)
    with open(d / "config.json", "w") as f:
        json.dump(tiny_config_json("A"), f)
    return str(d)


def test_a_tensor_in_two_shards_is_an_error_not_the_last_one_read(model_dirs, tmp_path):
    raw = load_file(os.path.join(model_dirs["A"], "model.safetensors"))
    names = sorted(raw)
    half = len(names) // 2
    twice = "model.layers.1.self_attn.o_proj.weight"
    first = {k: raw[k] for k in names[:half]}
    second = {k: raw[k] for k in names[half:]}
    first[twice] = raw[twice]
    second[twice] = torch.zeros_like(raw[twice])  # a stale copy: loading it silently would give wrong weights
    d = _folder_with(tmp_path, "dup", {"model-00001-of-00002.safetensors": first,
                                       "model-00002-of-00002.safetensors": second})
    with pytest.raises(WeightsError) as ei:
        load_model(d, "float32", "cpu")
    e = ei.value
    assert [n for n, _, _ in e.duplicate] == [twice]
    assert not e.missing and not e.unexpected and not e.wrong_shape
    assert "met twice (1)" in str(e) and "model-00001-of-00002.safetensors" in str(e) \
        and "model-00002-of-00002.safetensors" in str(e)


def test_a_tensor_with_and_without_the_optional_prefix_is_an_error(model_dirs, tmp_path):
    raw = load_file(os.path.join(model_dirs["A"], "model.safetensors"))
    raw["language_model.model.norm.weight"] = raw["model.norm.weight"] * 2
    d = _folder_with(tmp_path, "dup2", {"model.safetensors": raw})
    with pytest.raises(WeightsError) as ei:
        load_model(d, "float32", "cpu")
    assert [n for n, _, _ in ei.value.duplicate] == ["model.norm.weight"]
    assert "language_model.model.norm.weight" in str(ei.value)

"""Weights: safetensors round trip, binding by name, one error for every fault, the random-weights mode."""
import json
import os

import pytest
import torch

from atoma_infer_amd.config import load_model_config
from atoma_infer_amd.weights import (Checkpoint, SafetensorsFile, WeightsError, check_checkpoint, device_dtype_of,
                                     expected_tensors, write_random_model, write_safetensors)
from util import TINY_A, TINY_B, plain_weights


def test_safetensors_round_trip_and_the_package_agrees(tmp_path):
    ts = [("a", torch.randn(3, 5)), ("b.c", torch.randn(7).to(torch.bfloat16)),
          ("i", torch.arange(6, dtype=torch.int32).reshape(2, 3)), ("empty", torch.zeros(0, 4))]
    path = str(tmp_path / "x.safetensors")
    write_safetensors(path, ts, metadata={"seed": 3})
    f = SafetensorsFile(path)
    assert sorted(f.names()) == sorted(n for n, _ in ts) and f.metadata["seed"] == "3"
    for n, t in ts:
        assert f.dtype(n) is t.dtype and tuple(f.shape(n)) == tuple(t.shape)
        assert torch.equal(f.tensor(n), t)
    from safetensors.torch import load_file
    theirs = load_file(path)
    for n, t in ts:
        assert torch.equal(theirs[n], t)


def test_truncated_or_foreign_files_are_refused(tmp_path):
    p = tmp_path / "model.safetensors"
    p.write_bytes(b"\x10\x00\x00\x00\x00\x00\x00\x00{bad json")
    with pytest.raises(WeightsError):
        Checkpoint(str(tmp_path))
    with pytest.raises(WeightsError):
        Checkpoint(str(tmp_path / "missing"))


def test_random_model_is_a_function_of_config_seed_and_name(tmp_path):
    a = write_random_model(str(tmp_path / "a"), TINY_A, seed=1)
    b = write_random_model(str(tmp_path / "b"), TINY_A, seed=1)
    c = write_random_model(str(tmp_path / "c"), TINY_A, seed=2)
    wa, wb, wc = plain_weights(a), plain_weights(b), plain_weights(c)
    assert set(wa) == set(wb) and all(torch.equal(wa[k], wb[k]) for k in wa)
    assert not torch.equal(wa["model.embed_tokens.weight"], wc["model.embed_tokens.weight"])
    assert "lm_head.weight" not in wa                                  # tied
    assert os.path.isfile(os.path.join(a, "config.json"))
    arch, cfg = load_model_config(a)
    check_checkpoint(arch.build(cfg), Checkpoint(a))
    # statistics of the draws: linears N(0, 0.02), norms exactly 1 without jitter
    q = wa["model.layers.0.self_attn.q_proj.weight"]
    assert abs(float(q.std()) - 0.02) < 0.002 and abs(float(q.mean())) < 0.002
    assert torch.equal(wa["model.norm.weight"], torch.ones(64))
    d = write_random_model(str(tmp_path / "d"), TINY_B, seed=1, dtype="float32", norm_jitter=0.1)
    wd = plain_weights(d)
    assert "lm_head.weight" in wd and wd["lm_head.weight"].shape == (1000, 96)
    n = wd["model.layers.2.input_layernorm.weight"]
    assert 0.05 < float(n.std()) < 0.2 and abs(float(n.mean()) - 1) < 0.05
    assert Checkpoint(d).dtype("model.norm.weight") is torch.float32


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    d = write_random_model(str(tmp_path / "m"), TINY_A, seed=1)
    w = {k: v.to(torch.bfloat16) for k, v in plain_weights(d).items()}
    del w["model.layers.1.mlp.up_proj.weight"]
    del w["model.norm.weight"]
    w["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(32, 64, dtype=torch.bfloat16)
    w["model.layers.7.extra.weight"] = torch.zeros(2)
    w["model.layers.0.mlp.down_proj.weight"] = torch.zeros(64, 160, dtype=torch.int32)
    write_safetensors(os.path.join(d, "model.safetensors"), w.items())
    arch, cfg = load_model_config(d)
    with pytest.raises(WeightsError) as e:
        check_checkpoint(arch.build(cfg), Checkpoint(d))
    err = e.value
    assert sorted(err.missing) == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.7.extra.weight"]
    assert [(n, got, want) for n, got, want in err.wrong_shape] == \
        [("model.layers.0.self_attn.k_proj.weight", (32, 64), (16, 64))]
    assert [n for n, _, _ in err.wrong_kind] == ["model.layers.0.mlp.down_proj.weight"]
    for needle in ("missing (2)", "unexpected (1)", "wrong shape (1)", "model.norm.weight", "[32, 64]"):
        assert needle in str(err)


def test_tied_checkpoints_may_carry_a_head_and_old_buffers(tmp_path):
    """The reference ignores lm_head.weight when tied (models/src/llama.rs:482-486)."""
    d = write_random_model(str(tmp_path / "m"), TINY_A, seed=1)
    w = {k: v.to(torch.bfloat16) for k, v in plain_weights(d).items()}
    w["lm_head.weight"] = w["model.embed_tokens.weight"].clone()
    w["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    write_safetensors(os.path.join(d, "model.safetensors"), w.items())
    arch, cfg = load_model_config(d)
    check_checkpoint(arch.build(cfg), Checkpoint(d))
    # untied: the head is required
    cfg_untied = dict(TINY_A, tie_word_embeddings=False)
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(cfg_untied, f)
    del w["lm_head.weight"]
    write_safetensors(os.path.join(d, "model.safetensors"), w.items())
    arch, cfg = load_model_config(d)
    with pytest.raises(WeightsError) as e:
        check_checkpoint(arch.build(cfg), Checkpoint(d))
    assert e.value.missing == ["lm_head.weight"]


def test_sharded_checkpoints_merge_by_name(tmp_path):
    d = write_random_model(str(tmp_path / "m"), TINY_A, seed=1)
    w = {k: v.to(torch.bfloat16) for k, v in plain_weights(d).items()}
    names = sorted(w)
    half = len(names) // 2
    write_safetensors(os.path.join(d, "model-00001-of-00002.safetensors"), [(n, w[n]) for n in names[:half]])
    write_safetensors(os.path.join(d, "model-00002-of-00002.safetensors"), [(n, w[n]) for n in names[half:]])
    os.remove(os.path.join(d, "model.safetensors"))
    wm = {n: ("model-00001-of-00002.safetensors" if i < half else "model-00002-of-00002.safetensors")
          for i, n in enumerate(names)}
    with open(os.path.join(d, "model.safetensors.index.json"), "w") as f:
        json.dump({"weight_map": wm}, f)
    arch, cfg = load_model_config(d)
    ck = Checkpoint(d)
    check_checkpoint(arch.build(cfg), ck)
    assert torch.equal(ck.tensor(names[-1]), w[names[-1]])


def test_device_dtypes():
    assert device_dtype_of(torch.bfloat16) is torch.bfloat16 and device_dtype_of(torch.float32) is torch.float32
    assert device_dtype_of(torch.float16) is torch.float32 and device_dtype_of(torch.int64) is torch.int32


def test_expected_tensor_names_are_the_checkpoints_own():
    """models/src/llama.rs:481-489, 414-421, 322-325, 372-374."""
    from atoma_infer_amd.config import LlamaConfig
    from atoma_infer_amd.models.llama import build_llama
    names = set(expected_tensors(build_llama(LlamaConfig.from_dict(TINY_B))))
    want = {"model.embed_tokens.weight", "model.norm.weight", "lm_head.weight"}
    for i in range(3):
        p = f"model.layers.{i}."
        want |= {p + "input_layernorm.weight", p + "post_attention_layernorm.weight"}
        want |= {p + f"self_attn.{x}_proj.weight" for x in "qkvo"}
        want |= {p + f"mlp.{x}_proj.weight" for x in ("gate", "up", "down")}
    assert names == want

"""Weights: the safetensors reader and writer, the by-name loader's one error, the dtype
policy, the random-weights mode."""
import json
import os

import pytest
import torch
from safetensors.torch import load_file, save_file

from helpers import TINY_A, TINY_B
from tq_kv_amd import Model
from tq_kv_amd.weights import WeightError, WeightFileError, load_folder, open_folder, target_dtype, write_file


def test_writer_and_reader_agree_with_the_safetensors_package(tmp_path):
    t = {"a": torch.randn(3, 5).to(torch.bfloat16), "b": torch.arange(7, dtype=torch.int32), "c": torch.randn(2, 2, 2)}
    write_file(str(tmp_path / "x.safetensors"), t)
    back = load_file(str(tmp_path / "x.safetensors"))
    assert set(back) == set(t) and all(torch.equal(back[k], t[k]) for k in t)
    save_file({k: v.contiguous() for k, v in t.items()}, str(tmp_path / "y.safetensors"))
    (tmp_path / "x.safetensors").unlink()
    mine = open_folder(str(tmp_path))
    assert set(mine) == set(t)
    for k in t:
        assert mine[k].dtype == t[k].dtype and mine[k].shape == tuple(t[k].shape) and torch.equal(mine[k].read(), t[k])


def test_folder_errors(tmp_path):
    with pytest.raises(WeightFileError, match="No .safetensors files found"):
        open_folder(str(tmp_path))
    (tmp_path / "bad.safetensors").write_bytes(b"\x05\x00")
    with pytest.raises(WeightFileError, match="too short"):
        open_folder(str(tmp_path))
    (tmp_path / "bad.safetensors").write_bytes((1 << 40).to_bytes(8, "little") + b"{}")
    with pytest.raises(WeightFileError, match="header length"):
        open_folder(str(tmp_path))


def _folder(tmp_path, cfg, seed=0, dtype=torch.bfloat16):
    return Model.write_random_folder(str(tmp_path / "m"), cfg, seed=seed, store_dtype=dtype)


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    folder = _folder(tmp_path, TINY_B)
    path = os.path.join(folder, "model.safetensors")
    t = load_file(path)
    del t["model.layers.1.self_attn.k_proj.bias"], t["lm_head.weight"]
    t["model.layers.0.mlp.up_proj.weight"] = torch.zeros(224, 95, dtype=torch.bfloat16)
    t["model.layers.2.rogue.weight"] = torch.zeros(3, dtype=torch.bfloat16)
    t["model.norm.weight"] = torch.zeros(96, dtype=torch.int32)
    save_file(t, path)
    model = Model.from_config_dict(TINY_B, "float32", "cpu")
    with pytest.raises(WeightError) as e:
        load_folder(folder, model.tensor_specs(), torch.float32, "cpu")
    with pytest.raises(WeightError) as whole:
        Model.from_dir(folder, dtype="float32", device="cpu")               # the same error from the loader inside the library
    assert str(whole.value) == str(e.value) and whole.value.missing == e.value.missing
    msg = str(e.value)
    assert "Missing tensor: model.layers.1.self_attn.k_proj.bias" in msg and "Missing tensor: lm_head.weight" in msg
    assert "Unexpected tensor: model.layers.2.rogue.weight" in msg
    assert "model.layers.0.mlp.up_proj.weight is [224, 95], expected [224, 96]" in msg
    assert "Wrong dtype: model.norm.weight" in msg
    assert e.value.missing == ["model.layers.1.self_attn.k_proj.bias", "lm_head.weight"]
    assert len(e.value.wrong_shape) == 1 and len(e.value.unexpected) == 1


def test_tied_model_refuses_a_head_and_untied_needs_one(tmp_path):
    folder = _folder(tmp_path, TINY_A)
    path = os.path.join(folder, "model.safetensors")
    t = load_file(path)
    assert "lm_head.weight" not in t
    t["lm_head.weight"] = t["model.embed_tokens.weight"].clone()
    save_file(t, path)
    model = Model.from_config_dict(TINY_A, "float32", "cpu")
    with pytest.raises(WeightError, match="Unexpected tensor: lm_head.weight"):
        load_folder(folder, model.tensor_specs(), torch.float32, "cpu")
    # on request the tensors a model does not use are named in a warning instead (the reference never looks them up);
    # what is missing or misshapen stays an error
    with pytest.warns(UserWarning, match="lm_head.weight"):
        got = Model.from_dir(folder, dtype="float32", device="cpu", strict=False)
    assert got.head_is_embedding and not got.holds("lm_head.weight")
    del t["model.norm.weight"]
    save_file(t, path)
    with pytest.raises(WeightError, match="Missing tensor: model.norm.weight") as e:
        Model.from_dir(folder, dtype="float32", device="cpu", strict=False)
    assert "Unexpected" not in str(e.value)


def test_dtype_policy(tmp_path):
    bf, f32, f16 = torch.bfloat16, torch.float32, torch.float16
    assert target_dtype(bf, "float", bf) == bf and target_dtype(f16, "float", bf) == bf
    assert target_dtype(f32, "float", bf) == f32                  # stored in 32-bit stays so
    assert target_dtype(bf, "float", f32) == f32 and target_dtype(f16, "float", f32) == f32
    assert target_dtype(torch.int64, "int32", bf) == torch.int32
    folder = _folder(tmp_path, TINY_A)
    path = os.path.join(folder, "model.safetensors")
    t = load_file(path)
    t["model.norm.weight"] = t["model.norm.weight"].to(f32) + 1e-4     # not representable in bf16
    save_file(t, path)
    model = Model.from_config_dict(TINY_A, "bfloat16", "cpu")
    got = load_folder(folder, model.tensor_specs(), bf, "cpu")
    assert got["model.norm.weight"].dtype == f32 and torch.equal(got["model.norm.weight"], t["model.norm.weight"])
    assert got["model.embed_tokens.weight"].dtype == bf
    got = load_folder(folder, model.tensor_specs(), f32, "cpu")
    assert all(v.dtype == f32 for v in got.values())
    assert torch.equal(got["model.embed_tokens.weight"], t["model.embed_tokens.weight"].to(f32))
    # and what the library's own loader keeps, in host memory here
    kept = Model.from_dir(folder, dtype="bfloat16", device="cpu")
    assert kept.tensor("model.norm.weight").dtype == f32 and torch.equal(kept.tensor("model.norm.weight"), t["model.norm.weight"])
    assert kept.tensor("model.embed_tokens.weight").dtype == bf
    assert torch.equal(kept.tensor("model.embed_tokens.weight"), t["model.embed_tokens.weight"])
    kept = Model.from_dir(folder, dtype="float32", device="cpu")
    assert torch.equal(kept.tensor("model.embed_tokens.weight"), t["model.embed_tokens.weight"].to(f32))
    assert torch.equal(kept.tensor("model.layers.1.mlp.down_proj.weight"), t["model.layers.1.mlp.down_proj.weight"].to(f32))
    qkv = torch.cat([t["model.layers.0.self_attn.%s_proj.weight" % x] for x in "qkv"]).to(f32)
    assert torch.equal(kept.tensor("model.layers.0.self_attn.qkv.weight"), qkv)


def test_random_folder_is_seeded_and_has_the_stated_distributions(tmp_path):
    a = load_file(os.path.join(Model.write_random_folder(str(tmp_path / "a"), TINY_B, seed=1), "model.safetensors"))
    b = load_file(os.path.join(Model.write_random_folder(str(tmp_path / "b"), TINY_B, seed=1), "model.safetensors"))
    c = load_file(os.path.join(Model.write_random_folder(str(tmp_path / "c"), TINY_B, seed=2), "model.safetensors"))
    assert set(a) == set(Model.from_config_dict(TINY_B, "float32", "cpu").tensor_specs())
    assert all(torch.equal(a[k], b[k]) for k in a)
    assert not torch.equal(a["lm_head.weight"], c["lm_head.weight"])
    assert json.load(open(tmp_path / "a" / "config.json")) == TINY_B
    w = a["model.embed_tokens.weight"].float()
    assert abs(w.mean().item()) < 2e-3 and w.std().item() == pytest.approx(0.02, rel=0.05)
    n = a["model.layers.0.input_layernorm.weight"].float()
    assert n.mean().item() == pytest.approx(1.0, abs=0.01) and n.std().item() == pytest.approx(0.02, rel=0.3)
    bias = a["model.layers.2.self_attn.q_proj.bias"].float()
    assert bias.std().item() == pytest.approx(0.02, rel=0.3)
    # a tensor's stream depends on the seed and its name only, not on the other tensors
    tied = load_file(os.path.join(Model.write_random_folder(str(tmp_path / "d"), dict(TINY_B, tie_word_embeddings=True), seed=1),
                                  "model.safetensors"))
    assert "lm_head.weight" not in tied and torch.equal(tied["model.norm.weight"], a["model.norm.weight"])


def test_random_stream_is_a_function_of_key_and_index_alone():
    """Element i is the same whatever piece of the stream is asked for; the values are standard
    normal (moments and a Kolmogorov-Smirnov distance), bounded by sqrt(48 ln 2), never NaN."""
    import numpy as np
    from tq_kv_amd.weights import standard_normal_host, tensor_key
    key = tensor_key(3, "model.embed_tokens.weight")
    assert key == tensor_key(3, "model.embed_tokens.weight") != tensor_key(4, "model.embed_tokens.weight")
    whole = standard_normal_host(key, 0, 5000)
    pieces = np.concatenate([standard_normal_host(key, 0, 1), standard_normal_host(key, 1, 1999), standard_normal_host(key, 2000, 3000)])
    assert whole.dtype == np.float32 and np.array_equal(whole.view(np.int32), pieces.view(np.int32))
    assert not np.array_equal(whole, standard_normal_host(key + 1, 0, 5000))
    z = standard_normal_host(key, 0, 400000).astype(np.float64)
    assert np.isfinite(z).all() and np.abs(z).max() < 5.78
    assert abs(z.mean()) < 0.006 and abs(z.std() - 1) < 0.005 and abs((z ** 3).mean()) < 0.02 and abs((z ** 4).mean() - 3) < 0.05
    from scipy import stats
    assert stats.kstest(z, "norm").statistic < 0.003


def test_model_lists_tensors_by_the_reference_names():
    names = set(Model.from_config_dict(TINY_A, "float32", "cpu").tensor_specs())
    want = {"model.embed_tokens.weight", "model.norm.weight"}
    for l in range(2):
        p = "model.layers.%d." % l
        want |= {p + "self_attn.%s_proj.weight" % x for x in "qkvo"} | {p + "self_attn.%s_proj.bias" % x for x in "qkv"}
        want |= {p + "mlp.%s_proj.weight" % x for x in ("gate", "up", "down")}
        want |= {p + "input_layernorm.weight", p + "post_attention_layernorm.weight"}
    assert names == want


def test_packed_copy_of_a_weight_holds_every_value_once():
    """The few-row kernels' order: [tile of 16 rows][k / 32][lane][8], lane = 16 * ((k % 32) / 8) + row % 16,
    rows padded with zeros to whole tiles, stacked parts padded one by one."""
    from tq_kv_amd import kernels as K
    n, k = 40, 96
    w = torch.arange(n * k, dtype=torch.float32).reshape(n, k).to(torch.bfloat16)
    packed = K.pack_weight(w)
    assert tuple(packed.data.shape) == (3, 3, 64, 8) and packed.shape == (n, k) and packed.parts == 1
    for row in range(n):
        for col in range(0, k, 7):
            lane = 16 * ((col % 32) // 8) + row % 16
            assert packed.data[row // 16, col // 32, lane, col % 8] == w[row, col]
    assert packed.data.float().sum() == w.float().sum()         # the padding is zeros
    two = K.pack_weight(torch.cat([w, -w]), parts=2)
    assert tuple(two.data.shape) == (6, 3, 64, 8) and torch.equal(two.data[3:], -packed.data)
    with pytest.raises(K.KernelError, match="multiple of 32"):
        K.pack_weight(torch.zeros(16, 48, dtype=torch.bfloat16))
    with pytest.raises(K.KernelError, match="bfloat16"):
        K.pack_weight(torch.zeros(16, 64))

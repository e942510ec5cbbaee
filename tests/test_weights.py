"""Weights: the safetensors container, the check of a folder against what the model
expects (one error that lists everything), the type policy, and the random-weights mode."""
import json
import os
import struct

import pytest
import torch

import common
import llama_cu_amd
from llama_cu_amd.config import LlamaConfig
from llama_cu_amd.models.llama import llama_spec
from llama_cu_amd.parts import DecoderModel, TensorSpec
from llama_cu_amd.weights import (SafetensorsError, WeightError, check_tensors, load_weights, open_safetensors,
                                  random_tensors, write_random_model, write_safetensors)
from llama_cu_amd.weights.loader import convert


def expected(cfg_dict):
    return DecoderModel(llama_spec(LlamaConfig.from_dict(cfg_dict))).tensors()


def test_expected_tensor_names_and_shapes():
    e = expected(common.TINY_B)            # 3 layers, d 128, 4 heads of 32, 1 kv head, di 352, vocab 384, tied
    assert e["model.embed_tokens.weight"].shape == (384, 128)
    assert e["model.layers.2.self_attn.q_proj.weight"].shape == (128, 128)
    assert e["model.layers.0.self_attn.k_proj.weight"].shape == (32, 128)
    assert e["model.layers.0.self_attn.v_proj.weight"].shape == (32, 128)
    assert e["model.layers.1.self_attn.o_proj.weight"].shape == (128, 128)
    assert e["model.layers.1.mlp.gate_proj.weight"].shape == (352, 128)
    assert e["model.layers.1.mlp.up_proj.weight"].shape == (352, 128)
    assert e["model.layers.1.mlp.down_proj.weight"].shape == (128, 352)
    assert e["model.layers.1.input_layernorm.weight"].shape == (128,)
    assert e["model.layers.1.post_attention_layernorm.weight"].shape == (128,)
    assert e["model.norm.weight"].shape == (128,)
    assert e["lm_head.weight"].optional
    assert len(e) == 3 * 9 + 3


def test_container_round_trip_and_agreement_with_the_safetensors_package(tmp_path):
    tensors = {"a": torch.randn(3, 5), "b": torch.randn(7).to(torch.bfloat16), "c": torch.arange(6, dtype=torch.int32).view(2, 3),
               "empty": torch.zeros(0, 4)}
    path = str(tmp_path / "x.safetensors")
    write_safetensors(path, tensors)
    from llama_cu_amd.weights.safetensors_io import SafetensorsFile
    f = SafetensorsFile(path)
    assert sorted(f.names()) == sorted(tensors)
    for k, v in tensors.items():
        assert f.dtype(k) == v.dtype and f.shape(k) == tuple(v.shape) and torch.equal(f.tensor(k), v)
    from safetensors.torch import load_file, save_file
    theirs = load_file(path)                                   # their reader reads our file
    assert all(torch.equal(theirs[k], v) for k, v in tensors.items())
    path2 = str(tmp_path / "y.safetensors")
    save_file({k: v for k, v in tensors.items() if v.numel()}, path2)
    g = SafetensorsFile(path2)                                 # our reader reads their file
    assert all(torch.equal(g.tensor(k), tensors[k]) for k in g.names())


def test_broken_files_are_refused(tmp_path):
    path = str(tmp_path / "model.safetensors")
    write_safetensors(path, {"a": torch.randn(4, 4)})
    raw = open(path, "rb").read()
    open(path, "wb").write(raw[:-8])                           # truncated
    with pytest.raises(SafetensorsError, match="outside the file"):
        open_safetensors(str(tmp_path))
    open(path, "wb").write(struct.pack("<Q", 10 ** 9) + b"{}")
    with pytest.raises(SafetensorsError, match="header length"):
        open_safetensors(str(tmp_path))
    open(path, "wb").write(struct.pack("<Q", 5) + b"{oops")
    with pytest.raises(SafetensorsError, match="JSON"):
        open_safetensors(str(tmp_path))
    # header entries without their keys
    for entry, what in (({"dtype": "F32", "data_offsets": [0, 4]}, "shape"), ({"dtype": "F32", "shape": [1]}, "data_offsets"),
                        ({"dtype": "F32", "shape": [1], "data_offsets": [0]}, "data_offsets"), ("F32", "no object")):
        blob = json.dumps({"a": entry}).encode()
        open(path, "wb").write(struct.pack("<Q", len(blob)) + blob + b"\0" * 4)
        with pytest.raises(SafetensorsError, match=what):
            open_safetensors(str(tmp_path))
    os.remove(path)
    with pytest.raises(SafetensorsError, match="no model.safetensors"):
        open_safetensors(str(tmp_path))
    # an index that names a file that is not there, and one that is no index
    index = os.path.join(str(tmp_path), "model.safetensors.index.json")
    json.dump({"weight_map": {"a": "model-00001-of-00002.safetensors", "b": "model-00002-of-00002.safetensors"}}, open(index, "w"))
    write_safetensors(os.path.join(str(tmp_path), "model-00001-of-00002.safetensors"), {"a": torch.zeros(2)})
    with pytest.raises(SafetensorsError, match="model-00002-of-00002.safetensors"):
        open_safetensors(str(tmp_path))
    json.dump({"weights": {}}, open(index, "w"))
    with pytest.raises(SafetensorsError, match="weight_map"):
        open_safetensors(str(tmp_path))


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    folder = common.make_folder(common.TINY_A, seed=1, dtype=torch.float32, folder=str(tmp_path))
    from llama_cu_amd.weights.safetensors_io import SafetensorsFile
    w = {n: SafetensorsFile(os.path.join(folder, "model.safetensors")).tensor(n).clone()
         for n in SafetensorsFile(os.path.join(folder, "model.safetensors")).names()}
    del w["model.layers.1.mlp.up_proj.weight"]
    del w["model.norm.weight"]
    w["model.layers.0.self_attn.q_proj.weight"] = torch.zeros(64, 63)
    w["model.layers.7.extra.weight"] = torch.zeros(2)
    w["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)      # carried by some files, holds no weight
    write_safetensors(os.path.join(folder, "model.safetensors"), w)
    # which tensors a file may hold beside the weights is the architecture's business: its registry entry names them
    from llama_cu_amd.config import architecture_of
    ignored = architecture_of(common.TINY_A).ignored_tensors
    assert ignored
    with pytest.raises(WeightError) as err:
        load_weights(open_safetensors(folder), expected(common.TINY_A), torch.float32, torch.device("cpu"), ignored=ignored)
    msg = str(err.value)
    assert "missing tensors (2)" in msg and "model.layers.1.mlp.up_proj.weight" in msg and "model.norm.weight" in msg
    assert "unexpected tensors (1)" in msg and "model.layers.7.extra.weight" in msg and "inv_freq" not in msg
    assert "wrong shapes (1)" in msg and "found [64, 63], expected [64, 64]" in msg
    # the loader itself knows no such tensor
    with pytest.raises(WeightError, match=r"unexpected tensors \(2\)"):
        load_weights(open_safetensors(folder), expected(common.TINY_A), torch.float32, torch.device("cpu"))


def test_tied_and_untied_output_matrix(tmp_path):
    # tied model: no lm_head.weight needed; present but unused is fine too
    folder = common.make_folder(common.TINY_B, seed=1, dtype=torch.float32, folder=str(tmp_path))
    t = load_weights(open_safetensors(folder), expected(common.TINY_B), torch.float32, torch.device("cpu"))
    assert "lm_head.weight" not in t
    # an untied configuration whose file holds no output matrix falls back to the table
    # (the reference's rule, llama.cu/src/model/mod.rs:83-88): no error at load
    check_tensors(expected(dict(common.TINY_B, tie_word_embeddings=False)), {n: tuple(v.shape) for n, v in t.items()})


def test_type_policy():
    spec = TensorSpec((2, 2))
    f32, bf16, f16 = torch.ones(2, 2), torch.ones(2, 2, dtype=torch.bfloat16), torch.ones(2, 2, dtype=torch.float16)
    # bfloat16 engine: bfloat16 stays, 16-bit float becomes bfloat16, what is stored in 32-bit stays 32-bit
    assert convert(bf16, spec, torch.bfloat16).dtype == torch.bfloat16
    assert convert(f16, spec, torch.bfloat16).dtype == torch.bfloat16
    assert convert(f32, spec, torch.bfloat16).dtype == torch.float32
    # float32 engine: everything 32-bit, exactly
    x = torch.randn(2, 2).to(torch.bfloat16)
    assert torch.equal(convert(x, spec, torch.float32), x.float())
    assert convert(f32, spec, torch.float32).dtype == torch.float32
    # integer tables are int32
    ispec = TensorSpec((2, 2), integer=True)
    assert convert(torch.ones(2, 2, dtype=torch.int64), ispec, torch.bfloat16).dtype == torch.int32
    with pytest.raises(WeightError):
        convert(f32, ispec, torch.bfloat16)
    with pytest.raises(WeightError):
        convert(torch.ones(2, 2, dtype=torch.int32), spec, torch.bfloat16)


def test_random_weights_mode(tmp_path):
    cfg = LlamaConfig.from_dict(common.TINY_B)
    a = write_random_model(str(tmp_path / "a"), cfg, seed=5, dtype=torch.bfloat16)
    b = write_random_model(str(tmp_path / "b"), cfg, seed=5, dtype=torch.bfloat16)
    c = write_random_model(str(tmp_path / "c"), cfg, seed=6, dtype=torch.bfloat16)
    ra, rb, rc = (open(os.path.join(d, "model.safetensors"), "rb").read() for d in (a, b, c))
    assert ra == rb and ra != rc                                   # the seed decides
    assert LlamaConfig.from_dict(json.load(open(os.path.join(a, "config.json")))) == cfg
    t = load_weights(open_safetensors(a), expected(common.TINY_B), torch.bfloat16, torch.device("cpu"))
    assert "lm_head.weight" not in t                               # tied: none written
    q0, q1 = t["model.layers.0.self_attn.q_proj.weight"].float(), t["model.layers.1.self_attn.q_proj.weight"].float()
    assert not torch.equal(q0, q1)                                 # each tensor its own stream
    assert abs(float(q0.std()) - 0.02) < 0.002 and abs(float(q0.mean())) < 0.002
    n = t["model.norm.weight"].float()
    assert abs(float(n.mean()) - 1.0) < 0.01 and 0.01 < float(n.std()) < 0.03
    # a tensor's values do not depend on which other tensors the model has
    small = random_tensors({"model.norm.weight": TensorSpec((128,), init="one_plus_normal")}, 5, dtype=torch.bfloat16)
    assert torch.equal(small["model.norm.weight"], t["model.norm.weight"])
    # the plain implementation reads the folder too
    import plain
    pcfg, pw = plain.load_folder(a)
    assert plain.forward(pcfg, pw, [1, 2, 3]).shape == (3, 384)


def test_random_weights_of_an_untied_model_hold_an_output_matrix(tmp_path):
    cfg = LlamaConfig.from_dict(common.TINY_A)
    d = write_random_model(str(tmp_path / "a"), cfg, seed=1, dtype=torch.float32)
    t = load_weights(open_safetensors(d), expected(common.TINY_A), torch.float32, torch.device("cpu"))
    assert t["lm_head.weight"].shape == (256, 64)
    assert not torch.equal(t["lm_head.weight"], t["model.embed_tokens.weight"])


def test_random_model_command_writes_a_folder_that_loads(tmp_path):
    """``llama.cu_amd random-model CONFIG FOLDER --seed N``: the folder holds config.json and every
    tensor that the model expects, and the same seed gives the same bytes."""
    import json
    import llama_cu_amd.cli as cli
    cfg_path = tmp_path / "cfg.json"
    cfg_path.write_text(json.dumps(common.TINY_A))
    assert cli.main(["random-model", str(cfg_path), str(tmp_path / "m1"), "--seed", "4", "--dtype", "float32"]) == 0
    assert cli.main(["random-model", str(cfg_path), str(tmp_path / "m2"), "--seed", "4", "--dtype", "float32"]) == 0
    a = (tmp_path / "m1" / "model.safetensors").read_bytes()
    assert a == (tmp_path / "m2" / "model.safetensors").read_bytes()
    assert json.loads((tmp_path / "m1" / "config.json").read_text())["hidden_size"] == common.TINY_A["hidden_size"]
    files = open_safetensors(str(tmp_path / "m1"))
    names = {n for f in files for n in f.names()}
    assert "model.embed_tokens.weight" in names and "model.layers.1.mlp.down_proj.weight" in names



def test_the_generator_is_a_function_of_seed_name_and_index_and_is_normal():
    """Element i of a tensor depends on (seed, name, i) alone; the values are Box-Muller normals:
    a plain formula with the library's logarithm and cosine gives the same numbers to within the
    polynomials' error, and the moments of a million of them are those of N(0, 1)."""
    import math
    from llama_cu_amd.weights import fill_normal, stream_key
    key = stream_key(7, "model.embed_tokens.weight")
    assert key != stream_key(8, "model.embed_tokens.weight") and key != stream_key(7, "model.embed_tokens.weigh")
    assert stream_key(0, "a") != stream_key(1, "a") != stream_key(2, "a")
    t = fill_normal(torch.empty(1 << 20), key, 1.0)
    short = fill_normal(torch.empty(1000), key, 1.0)
    assert torch.equal(short, t[:1000])                              # a prefix of the same stream
    mask = (1 << 64) - 1

    def mix(z):
        z &= mask; z ^= z >> 30; z = z * 0xBF58476D1CE4E5B9 & mask; z ^= z >> 27; z = z * 0x94D049BB133111EB & mask
        return z ^ (z >> 31)
    for i in (0, 1, 2, 999, 12345, (1 << 20) - 1):
        z = mix(key + (i + 1) * 0x9E3779B97F4A7C15)
        u1, u2 = ((z >> 32) + 0.5) / 2 ** 32, ((z & 0xFFFFFFFF) + 0.5) / 2 ** 32
        want = math.sqrt(-2 * math.log(u1)) * math.cos(2 * math.pi * u2)
        assert abs(float(t[i]) - want) <= 1e-6 * max(1.0, abs(want)), (i, float(t[i]), want)
    d = t.double()
    assert abs(float(d.mean())) < 4e-3 and abs(float(d.std()) - 1) < 4e-3
    assert abs(float((d ** 3).mean())) < 2e-2 and abs(float((d ** 4).mean()) - 3) < 5e-2
    assert 4.0 < float(d.abs().max()) < 6.5                           # tails are there, and finite
    assert abs(float((d[1:] * d[:-1]).mean())) < 4e-3                  # neighbours are uncorrelated
    # scale and shift in 32-bit, one rounding to bfloat16
    f = fill_normal(torch.empty(4096), key, 0.02, 1.0)
    assert torch.equal(f, t[:4096] * 0.02 + 1.0)
    assert torch.equal(fill_normal(torch.empty(4096, dtype=torch.bfloat16), key, 0.02, 1.0), f.to(torch.bfloat16))
    with pytest.raises(ValueError):
        fill_normal(torch.empty(4, dtype=torch.float16), key, 1.0)


def test_weights_lie_in_one_allocation_and_fused_tensors_stand_in_place(tmp_path):
    """All tensors are views of one allocation; q, k, v and gate, up stand one after the other, so
    that the fused matrices are views too (nothing is concatenated), also when the file stores
    another type than the engine keeps; with rows of zeros behind each member where asked for."""
    from llama_cu_amd.models.llama import llama_spec
    from llama_cu_amd.parts import DecoderModel
    from llama_cu_amd.weights.loader import FusedGroup, fused_rows, plan_arena
    cfg = LlamaConfig.from_dict(common.TINY_B)
    model = DecoderModel(llama_spec(cfg))
    groups = model.fused_groups(torch.bfloat16, torch.device("cpu"))
    assert FusedGroup(("model.layers.1.self_attn.q_proj.weight", "model.layers.1.self_attn.k_proj.weight",
                       "model.layers.1.self_attn.v_proj.weight"), 0) in groups
    assert FusedGroup(("model.layers.2.mlp.gate_proj.weight", "model.layers.2.mlp.up_proj.weight"), 0) in groups
    lines = []
    for stored, compute in ((torch.float16, torch.bfloat16), (torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16)):
        folder = write_random_model(str(tmp_path / f"m{len(lines)}"), cfg, seed=3, dtype=stored, vector_dtype=torch.float32)
        t = load_weights(open_safetensors(folder), model.tensors(), compute, torch.device("cpu"), groups=groups, log=lines.append)
        base = {v.untyped_storage().data_ptr() for v in t.values()}
        assert len(base) == 1                                                # one allocation
        start = next(iter(base))
        assert all((v.data_ptr() - start) % 256 == 0 or "k_proj" in n or "v_proj" in n or "up_proj" in n for n, v in t.items())
        p = "model.layers.0."
        q, k, v = (t[p + f"self_attn.{x}_proj.weight"] for x in "qkv")
        qkv = fused_rows([q, k, v])
        assert qkv.data_ptr() == q.data_ptr() and qkv.shape == (q.shape[0] + k.shape[0] + v.shape[0], 128)
        assert torch.equal(qkv, torch.cat([q, k, v]))
        gu = fused_rows([t[p + "mlp.gate_proj.weight"], t[p + "mlp.up_proj.weight"]])
        assert gu.data_ptr() == t[p + "mlp.gate_proj.weight"].data_ptr()
        assert t["model.norm.weight"].dtype == torch.float32                 # stored in 32-bit: stays so
        assert q.dtype == compute
        # the values are the file's, converted once
        raw = open_safetensors(folder)[0].tensor(p + "self_attn.k_proj.weight")
        assert torch.equal(k, raw.to(compute))
    assert len(lines) == 3 and "GB/s" in lines[0] and "one allocation" in lines[0]
    # tensors that do not stand together are concatenated, with the same result
    a, b = torch.randn(3, 8), torch.randn(5, 8)
    assert torch.equal(fused_rows([a, b]), torch.cat([a, b]))
    assert fused_rows([a, b], pad_rows_to=6).shape == (12, 8) and bool((fused_rows([a, b], pad_rows_to=6)[3:6] == 0).all())
    # rows of zeros behind each member of a group
    expected = {"g": TensorSpec((5, 8)), "u": TensorSpec((5, 8)), "x": TensorSpec((3,))}
    place, total = plan_arena(expected, {n: torch.bfloat16 for n in expected}, torch.bfloat16, [FusedGroup(("g", "u"), 8)])
    assert place["u"][0] - place["g"][0] == 8 * 8 * 2 and place["x"][0] >= place["u"][0] + 8 * 8 * 2 and total % 256 == 0


def test_a_part_names_how_its_tensors_start_and_may_bring_its_own_way():
    """``TensorSpec.init`` names an initialiser of a registry: zeros and ones are there beside the two normal ones, a
    part from outside registers its own (here a decay spread evenly over a range, made from the tensor's own stream),
    and a name that nothing registers is an error that lists the registered ones."""
    from llama_cu_amd.weights import fill_normal, random_tensors, register_initialiser, registered_initialisers

    def decay(out, key, std):
        fill_normal(out, key, 1.0)                              # the tensor's stream: the same bits on host and GPU
        out.copy_(torch.sigmoid(out.float()) * 0.5 + 0.4)       # into (0.4, 0.9)

    register_initialiser("toy_decay", decay, replace=True)
    assert {"normal", "one_plus_normal", "zeros", "ones", "toy_decay"} <= set(registered_initialisers())
    want = {"a.weight": TensorSpec((8, 16)), "a.bias": TensorSpec((8,), init="zeros"), "a.gain": TensorSpec((8,), init="ones"),
            "a.decay": TensorSpec((64,), init="toy_decay")}
    t = random_tensors(want, 5, dtype=torch.float32, std=0.02)
    assert float(t["a.bias"].abs().max()) == 0.0 and bool((t["a.gain"] == 1.0).all())
    assert 0.4 < float(t["a.decay"].min()) and float(t["a.decay"].max()) < 0.9 and float(t["a.decay"].std()) > 0.05
    assert 0.01 < float(t["a.weight"].std()) < 0.03
    again = random_tensors(want, 5, dtype=torch.float32, std=0.02)
    assert all(torch.equal(t[k], again[k]) for k in t)
    with pytest.raises(ValueError, match="registered"):
        random_tensors({"b.weight": TensorSpec((2, 2), init="no_such_start")}, 1)
    with pytest.raises(ValueError, match="already registered"):
        register_initialiser("zeros", decay)

import json
import os

import pytest
import torch

from conftest import TINY, TINY_A
from denno_beta_amd.config import load_config
from denno_beta_amd.weights import (CheckpointError, SafetensorsFile, load_checkpoint, write_model_folder,
                                    write_safetensors)


def specs_of(folder):
    arch, cfg = load_config(folder)
    return arch.build(cfg)


def rewrite(folder, change):
    """Rewrites model.safetensors after `change(dict of tensors)`."""
    from safetensors.torch import load_file, save_file
    path = os.path.join(folder, "model.safetensors")
    t = load_file(path)
    change(t)
    save_file({k: v.contiguous() for k, v in t.items()}, path)


def load(folder, dtype="float32", **kw):
    spec = specs_of(folder)
    return load_checkpoint(folder, spec.param_specs(), engine_dtype=dtype, device="cpu",
                           prefixes=spec.name_prefixes, ignore=spec.ignore_tensors, tied=spec.tied_tensors, **kw)


def test_random_folder_reads_back_and_matches_the_library_reader(tmp_path):
    from safetensors.torch import load_file
    d = write_model_folder(str(tmp_path / "m"), TINY_A, seed=0)
    ours = SafetensorsFile(os.path.join(d, "model.safetensors"))
    theirs = load_file(os.path.join(d, "model.safetensors"))
    assert set(ours.entries) == set(theirs)
    for name in theirs:
        assert torch.equal(ours.tensor(name), theirs[name])
    # names and shapes as the reference reads them (gpt2.rs:70-83, 112-115): Conv1D is [in, out]
    assert tuple(theirs["h.0.attn.c_attn.weight"].shape) == (64, 192)
    assert tuple(theirs["h.1.mlp.c_proj.weight"].shape) == (256, 64)
    assert tuple(theirs["wte.weight"].shape) == (512, 64) and tuple(theirs["wpe.weight"].shape) == (128, 64)
    assert abs(theirs["h.0.ln_1.weight"].mean().item() - 1.0) < 0.02
    assert abs(theirs["h.0.attn.c_attn.weight"].std().item() - 0.02) < 0.002
    assert abs(theirs["h.0.attn.c_attn.bias"].std().item() - 0.01) < 0.003


def test_values_depend_on_seed_and_name_only(tmp_path):
    from safetensors.torch import load_file
    a = load_file(os.path.join(write_model_folder(str(tmp_path / "a"), TINY_A, seed=3), "model.safetensors"))
    b = load_file(os.path.join(write_model_folder(str(tmp_path / "b"), TINY_A, seed=3), "model.safetensors"))
    c = load_file(os.path.join(write_model_folder(str(tmp_path / "c"), TINY_A, seed=4), "model.safetensors"))
    more = load_file(os.path.join(write_model_folder(str(tmp_path / "d"), dict(TINY_A, n_layer=3), seed=3),
                                  "model.safetensors"))
    for n in a:
        assert torch.equal(a[n], b[n]) and torch.equal(a[n], more[n])
    assert not torch.equal(a["wte.weight"], c["wte.weight"])


def test_held_layout_and_dtypes(tmp_path):
    d = write_model_folder(str(tmp_path / "m"), TINY_A, seed=0, dtype="bfloat16")
    t16 = load(d, "bfloat16")
    assert t16["h.0.attn.c_attn.weight"].dtype == torch.bfloat16
    assert tuple(t16["h.0.attn.c_attn.weight"].shape) == (192, 64)       # held [out, in]
    assert t16["h.0.attn.c_attn.bias"].dtype == torch.float32           # vectors are held in 32-bit
    assert t16["h.0.ln_1.weight"].dtype == torch.float32 and t16["wte.weight"].dtype == torch.bfloat16
    t32 = load(d, "float32")
    assert all(v.dtype == torch.float32 for v in t32.values())
    assert torch.equal(t32["wte.weight"], t16["wte.weight"].float())     # widening is exact
    # a folder stored in 32-bit stays 32-bit in a bfloat16 engine, unless asked to be rounded
    d32 = write_model_folder(str(tmp_path / "m32"), TINY_A, seed=0, dtype="float32")
    notes = []
    kept = load(d32, "bfloat16", notes=notes)
    assert kept["h.0.attn.c_attn.weight"].dtype == torch.float32 and notes
    cast = load(d32, "bfloat16", cast_matrices=True)
    assert cast["h.0.attn.c_attn.weight"].dtype == torch.bfloat16 and cast["ln_f.bias"].dtype == torch.float32


def test_prefix_buffers_and_tied_head_are_accepted(tmp_path):
    d = write_model_folder(str(tmp_path / "m"), TINY_A, seed=0)
    plain = load(d)

    def change(t):
        for k in list(t):
            t["transformer." + k] = t.pop(k)
        t["lm_head.weight"] = t["transformer.wte.weight"].clone()
        t["transformer.h.0.attn.bias"] = torch.ones(1, 1, 128, 128)
        t["transformer.h.1.attn.masked_bias"] = torch.tensor(-1e4)
    rewrite(d, change)
    again = load(d)
    assert set(again) == set(plain) and all(torch.equal(again[k], plain[k]) for k in plain)


def test_one_error_lists_everything(tmp_path):
    d = write_model_folder(str(tmp_path / "m"), TINY_A, seed=0)

    def change(t):
        del t["h.1.ln_2.bias"]
        del t["wpe.weight"]
        t["h.0.mlp.c_fc.weight"] = torch.zeros(64, 128)
        t["h.7.attn.c_attn.weight"] = torch.zeros(2, 2)
        t["extra.thing"] = torch.zeros(3)
    rewrite(d, change)
    with pytest.raises(CheckpointError) as ei:
        load(d)
    e = ei.value
    assert sorted(e.missing) == ["h.1.ln_2.bias", "wpe.weight"]
    assert sorted(e.unexpected) == ["extra.thing", "h.7.attn.c_attn.weight"]
    assert [(n, tuple(g), tuple(w)) for n, g, w in e.wrong_shape] == [("h.0.mlp.c_fc.weight", (64, 128), (64, 256))]
    msg = str(e)
    for word in ("missing", "unexpected", "wrong shapes", "wpe.weight", "extra.thing", "h.0.mlp.c_fc.weight"):
        assert word in msg


def test_wrong_dtype_and_broken_files(tmp_path):
    d = write_model_folder(str(tmp_path / "m"), TINY_A, seed=0)
    rewrite(d, lambda t: t.__setitem__("wte.weight", torch.zeros(512, 64, dtype=torch.int32)))
    with pytest.raises(CheckpointError, match="unsupported dtypes"):
        load(d)
    empty = tmp_path / "none"
    empty.mkdir()
    (empty / "config.json").write_text(json.dumps(TINY_A))
    with pytest.raises(ValueError, match="model.safetensors"):
        load(str(empty))
    (empty / "model.safetensors").write_bytes(b"\x10\x00\x00\x00\x00\x00\x00\x00{bad")
    with pytest.raises(ValueError):
        load(str(empty))


def test_sharded_checkpoint(tmp_path):
    from safetensors.torch import load_file, save_file
    d = write_model_folder(str(tmp_path / "m"), TINY_A, seed=0)
    whole = load(d)
    t = load_file(os.path.join(d, "model.safetensors"))
    names = sorted(t)
    half = len(names) // 2
    save_file({n: t[n] for n in names[:half]}, os.path.join(d, "model-00001-of-00002.safetensors"))
    save_file({n: t[n] for n in names[half:]}, os.path.join(d, "model-00002-of-00002.safetensors"))
    os.remove(os.path.join(d, "model.safetensors"))
    wm = {n: ("model-00001-of-00002.safetensors" if i < half else "model-00002-of-00002.safetensors")
          for i, n in enumerate(names)}
    with open(os.path.join(d, "model.safetensors.index.json"), "w") as f:
        json.dump({"weight_map": wm}, f)
    shards = load(d)
    assert all(torch.equal(shards[k], whole[k]) for k in whole)


def test_streaming_writer_checks_its_layout(tmp_path):
    with pytest.raises(ValueError, match="layout says"):
        write_safetensors(str(tmp_path / "x.safetensors"), [("a", torch.float32, (2, 2))],
                          lambda n: torch.zeros(3))


def test_a_tensor_stored_in_pieces_is_joined_at_load(tmp_path):
    """A held tensor may be several file tensors joined along one dimension of the stored layout (a fused
    projection whose q, k and v a checkpoint stores apart): the pieces are read by their own names, joined in
    the spec's order, and everything wrong is reported by the file's names, all at once."""
    from denno_beta_amd.weights import ParamSpec
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(n, 6, generator=g) for n in (8, 4, 4))           # stored [out, in]
    qc, kc, vc = (torch.randn(6, n, generator=g) for n in (8, 4, 4))        # stored [in, out]
    bq, bk, bv = (torch.randn(n, generator=g) for n in (8, 4, 4))
    tensors = {"a.q": q, "a.k": k, "a.v": v, "c.q": qc, "c.k": kc, "c.v": vc, "a.bq": bq, "a.bk": bk, "a.bv": bv,
               "n.w": torch.ones(6)}
    specs = [ParamSpec("a.qkv", (16, 6), "matrix", sources=(("a.q", 8), ("a.k", 4), ("a.v", 4)), concat_dim=0),
             ParamSpec("c.qkv", (6, 16), "matrix", transpose=True, sources=(("c.q", 8), ("c.k", 4), ("c.v", 4)), concat_dim=1),
             ParamSpec("a.b", (16,), "vector", sources=(("a.bq", 8), ("a.bk", 4), ("a.bv", 4))),
             ParamSpec("n.w", (6,), "vector")]

    def write(d, t, dtype=torch.float32):
        os.makedirs(d, exist_ok=True)
        write_safetensors(os.path.join(d, "model.safetensors"),
                          [(n, torch.float32 if x.dim() == 1 else dtype, tuple(x.shape)) for n, x in t.items()],
                          lambda n: t[n].to(torch.float32 if t[n].dim() == 1 else dtype))
        return d
    d = write(str(tmp_path / "ok"), tensors)
    got = load_checkpoint(d, specs, engine_dtype="float32", device="cpu")
    assert set(got) == {"a.qkv", "c.qkv", "a.b", "n.w"}
    assert torch.equal(got["a.qkv"], torch.cat([q, k, v], 0))
    assert torch.equal(got["c.qkv"], torch.cat([qc, kc, vc], 1).t()) and got["c.qkv"].is_contiguous()
    assert torch.equal(got["a.b"], torch.cat([bq, bk, bv]))
    # bfloat16 pieces stay bfloat16 in a bfloat16 engine; one piece in 32-bit keeps the whole in 32-bit
    d = write(str(tmp_path / "bf"), tensors, torch.bfloat16)
    assert load_checkpoint(d, specs, engine_dtype="bfloat16", device="cpu")["a.qkv"].dtype == torch.bfloat16
    rewrite(d, lambda t: t.__setitem__("a.k", t["a.k"].float()))
    got = load_checkpoint(d, specs, engine_dtype="bfloat16", device="cpu")
    assert got["a.qkv"].dtype == torch.float32 and got["c.qkv"].dtype == torch.bfloat16
    # a missing piece, a piece of the wrong shape, the joined name itself in the file: one error
    bad = dict(tensors)
    del bad["a.k"]
    bad["c.v"] = torch.zeros(6, 5)
    bad["a.qkv"] = torch.zeros(16, 6)
    with pytest.raises(CheckpointError) as e:
        load_checkpoint(write(str(tmp_path / "bad"), bad), specs, engine_dtype="float32", device="cpu")
    assert e.value.missing == ["a.k"] and e.value.unexpected == ["a.qkv"]
    assert [(n, tuple(s), tuple(w)) for n, s, w in e.value.wrong_shape] == [("c.v", (6, 5), (6, 4))]
    # sizes that do not add up are a fault of the description
    with pytest.raises(ValueError, match="add up"):
        ParamSpec("x", (16, 6), "matrix", sources=(("a", 8), ("b", 4)))

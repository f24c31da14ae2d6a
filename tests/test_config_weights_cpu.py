"""Configuration, registry, weight loading errors and the random-weights writer (no GPU)."""

import json

import pytest
import torch
from safetensors.torch import load_file, save_file

from kestrel_amd.config import RuntimeConfig, get_spec, known_models, read_model_dir, resolve
from kestrel_amd.models import DecoderModel
from kestrel_amd.models.moondream import MoondreamTextConfig
from kestrel_amd.weights import InitRecipe, WeightsError, held_dtype, load_tensors, write_random_model
from tests import helpers


def test_registry_names_and_unknown_model():
    assert "moondream2" in known_models()
    assert get_spec("HfMoondream").name == "moondream2"
    with pytest.raises(ValueError, match=r"Unknown model 'nope'\. Known models: .*moondream2"):
        get_spec("nope")
    assert resolve({"model_type": "moondream1"}).name == "moondream2"
    assert resolve(helpers.TINY_A).name == "moondream2"       # claimed by its keys
    with pytest.raises(ValueError, match="names no architecture"):
        resolve({"hidden_size": 8})


def test_config_reads_every_key_and_derives_the_fixed_ones():
    cfg = MoondreamTextConfig.from_dict(helpers.TINY_B)
    assert (cfg.dim, cfg.ff_dim, cfg.n_layers, cfg.vocab_size, cfg.max_context) == (96, 320, 3, 1000, 256)
    assert (cfg.n_heads, cfg.n_kv_heads, cfg.head_dim, cfg.rotary_dim) == (3, 1, 32, 16)
    assert cfg.rope_theta == 5000.0 and cfg.layer_norm_eps == 1e-6 and cfg.prefix_attn == 17
    c = MoondreamTextConfig.from_dict(helpers.TINY_C)
    assert (c.head_dim, c.rotary_dim) == (48, 12)
    flat = MoondreamTextConfig.from_dict(dict(helpers.TINY_A["text"]))
    assert flat == MoondreamTextConfig.from_dict(helpers.TINY_A)
    assert flat.layer_norm_eps == 1e-5
    # a config.json without a text section is the released model (sizes from the preset file)
    released = MoondreamTextConfig.from_dict({"model_type": "moondream1", "config": {}})
    assert (released.dim, released.n_layers, released.vocab_size, released.head_dim) == (2048, 24, 51200, 64)
    assert MoondreamTextConfig.from_dict(released.to_dict()) == released


@pytest.mark.parametrize("change, message", [
    ({"dim": None}, "missing"), ({"n_heads": 5}, "no multiple"), ({"n_kv_heads": 3}, "no multiple of n_kv_heads"),
    ({"moe": {"num_experts": 4}}, "moe"), ({"tau_attn": True}, "tau"), ({"rotary_dim": 7}, "rotary_dim"),
    ({"vocab_size": -1}, "positive integer"), ({"bogus": 1}, "unknown text keys"), ({"layer_norm_eps": 0}, "positive"),
])
def test_config_errors(change, message):
    text = dict(helpers.TINY_A["text"])
    for key, value in change.items():
        if value is None:
            text.pop(key)
        else:
            text[key] = value
    with pytest.raises((ValueError, NotImplementedError), match=message):
        MoondreamTextConfig.from_dict({"text": text})


def test_other_spellings_of_the_added_keys():
    from kestrel_amd.config import get_spec
    from kestrel_amd.config.registry import resolve

    base = {k: v for k, v in helpers.flat_config("C").items() if k not in ("layer_norm_eps", "rotary_dim", "rope_theta")}
    spelled = dict(base, eps=3e-5, rope_dim=12, theta=1234.5)
    for config in (spelled, {"text": spelled}):
        assert resolve(config).name == "moondream2"
        cfg = get_spec("moondream2").read_config(config)
        assert (cfg.layer_norm_eps, cfg.rotary_dim, cfg.rope_theta) == (3e-5, 12, 1234.5)
    with pytest.raises(ValueError, match="name the same value"):
        get_spec("moondream2").read_config(dict(spelled, ln_eps=1e-5))
    with pytest.raises(ValueError, match="name the same value"):
        get_spec("moondream2").read_config(dict(spelled, layer_norm_eps=1e-5))


def test_quantized_config_is_refused():
    text = dict(helpers.TINY_A["text"], group_size=128)
    with pytest.raises(NotImplementedError):
        MoondreamTextConfig.from_dict({"text": text})


def test_plan_is_data():
    spec = get_spec("moondream2")
    plan = spec.build_plan(spec.read_config(helpers.TINY_C))
    assert len(plan.layers) == 2 and [e.layer for e in plan.schedule] == [0, 1]
    layer = plan.layers[1]
    assert layer.arrangement == "parallel" and layer.mixer.kind == "attention" and layer.feed_forward.kind == "dense"
    assert layer.mixer.head_dim == 48 and layer.mixer.position.rotary_dim == 12 and layer.norm.eps == 3e-5
    assert layer.names["mixer.qkv.weight"] == "text.blocks.1.attn.qkv.weight"
    params = DecoderModel(plan).params()
    assert params["text.blocks.0.attn.qkv.weight"].shape == ((6 + 2 * 2) * 48, 120)
    assert params["text.lm_head.weight"].shape == (777, 120) and params["text.wte"].shape == (777, 120)


def test_runtime_config_checks():
    cfg = RuntimeConfig(model_path="x", dtype="float32", kv_cache_pages=8)
    assert cfg.dtype == torch.float32 and cfg.page_size == 16
    for bad in (dict(kv_cache_pages=0), dict(max_batch_size=0), dict(dtype="float16"), dict(device="cpu"),
                dict(page_size=0), dict(max_num_batched_tokens=0), dict(kv_cache_bytes=0),
                dict(kv_cache_bytes=1 << 30, kv_cache_pages=8), dict(kv_cache_tokens=64, kv_cache_pages=8)):
        with pytest.raises(ValueError):
            RuntimeConfig(model_path="x", **bad)


def test_the_cache_pool_is_sized_by_pages_tokens_or_bytes():
    """``kv_cache_pages`` or ``kv_cache_bytes`` (``kestrel/kv_cache.py:52-136``: a byte budget, and
    ``MemoryError`` beyond it), or tokens; the default is ``max_batch_size`` full contexts. A pool that
    does not fit in what the device has free is refused before anything is allocated."""
    from kestrel_amd.engine.engine import pool_pages

    per_page = 3 * 1024 * 1024          # Moondream 2: 16 tokens x 196,608 bytes
    assert pool_pages(RuntimeConfig(model_path="x", kv_cache_pages=40), per_page, 2048, None) == 40
    assert pool_pages(RuntimeConfig(model_path="x", kv_cache_tokens=1000), per_page, 2048, None) == 63
    assert pool_pages(RuntimeConfig(model_path="x", kv_cache_bytes=60 * 10 ** 9), per_page, 2048, None) == 19073
    assert pool_pages(RuntimeConfig(model_path="x", max_batch_size=4), per_page, 2048, None) == 4 * 128
    with pytest.raises(MemoryError, match="holds less than one page"):
        pool_pages(RuntimeConfig(model_path="x", kv_cache_bytes=1000), per_page, 2048, None)
    # 512 pages of 3 MiB do not fit in 1 GiB free
    with pytest.raises(MemoryError, match="1.5 GiB.*1.0 GiB free"):
        pool_pages(RuntimeConfig(model_path="x", max_batch_size=4), per_page, 2048, 1 << 30)
    assert pool_pages(RuntimeConfig(model_path="x", max_batch_size=4), per_page, 2048, 4 << 30) == 512


def test_random_model_folder_roundtrip(tmp_path):
    folder = write_random_model(tmp_path / "m", helpers.TINY_B, seed=1, recipe=helpers.RECIPES["B"])
    spec, typed, plan = read_model_dir(folder)
    assert spec.name == "moondream2" and typed == MoondreamTextConfig.from_dict(helpers.TINY_B)
    stored = load_file(str(folder / "model.safetensors"))
    expected = DecoderModel(plan).params()
    assert set(stored) == set(expected)
    assert all(t.dtype == torch.bfloat16 for t in stored.values())
    gain = stored["text.blocks.0.ln.weight"].float()
    assert abs(gain.mean().item() - 1.0) < 0.02 and 0.005 < gain.std().item() < 0.05
    assert abs(stored["text.wte"].float().std().item() - 0.03) < 0.003
    # the same seed gives the same tensors whatever else is drawn; another seed does not
    again = write_random_model(tmp_path / "n", helpers.TINY_B, seed=1, recipe=helpers.RECIPES["B"])
    assert torch.equal(load_file(str(again / "model.safetensors"))["text.blocks.2.mlp.fc1.weight"],
                       stored["text.blocks.2.mlp.fc1.weight"])
    other = write_random_model(tmp_path / "o", helpers.TINY_B, seed=2, recipe=helpers.RECIPES["B"])
    assert not torch.equal(load_file(str(other / "model.safetensors"))["text.wte"], stored["text.wte"])


def _params(name="A"):
    spec = get_spec("moondream2")
    return spec, DecoderModel(spec.build_plan(spec.read_config(helpers.CONFIGS[name]))).params()


def test_loader_types():
    spec, params = _params()
    path = helpers.model_dir("A") + "/model.safetensors"
    bf = load_tensors(path, params, torch.bfloat16, prefixes=spec.tensor_prefixes)
    assert all(t.dtype == torch.bfloat16 for t in bf.values())
    fp = load_tensors(path, params, torch.float32, prefixes=spec.tensor_prefixes)
    assert all(t.dtype == torch.float32 for t in fp.values())
    assert torch.equal(fp["text.wte"], bf["text.wte"].float())
    assert held_dtype(torch.float32, "vector", torch.bfloat16) == torch.float32     # stored in 32 bits: stays so
    assert held_dtype(torch.float16, "matrix", torch.bfloat16) == torch.bfloat16
    assert held_dtype(torch.int64, "table", torch.bfloat16) == torch.int32


def test_loader_keeps_32_bit_tensors_and_accepts_the_checkpoint_prefix(tmp_path):
    spec, params = _params()
    stored = load_file(helpers.model_dir("A") + "/model.safetensors")
    renamed = {"model." + k: v for k, v in stored.items()}
    renamed["model.text.post_ln.weight"] = renamed["model.text.post_ln.weight"].float()
    renamed["model.vision.proj.weight"] = torch.zeros(3, 3)          # another part of the checkpoint: passed over
    path = tmp_path / "model.safetensors"
    save_file(renamed, str(path))
    got = load_tensors(path, params, torch.bfloat16, prefixes=spec.tensor_prefixes, foreign_prefixes=spec.foreign_prefixes)
    assert got["text.post_ln.weight"].dtype == torch.float32 and got["text.wte"].dtype == torch.bfloat16
    assert set(got) == set(params)


def test_loader_reports_everything_at_once(tmp_path):
    spec, params = _params()
    stored = load_file(helpers.model_dir("A") + "/model.safetensors")
    del stored["text.blocks.1.ln.bias"]
    del stored["text.lm_head.bias"]
    stored["text.blocks.0.mlp.fc1.weight"] = torch.zeros(8, 8, dtype=torch.bfloat16)
    stored["text.blocks.9.ln.weight"] = torch.zeros(64, dtype=torch.bfloat16)
    stored["stray"] = torch.zeros(1)
    path = tmp_path / "model.safetensors"
    save_file(stored, str(path))
    with pytest.raises(WeightsError) as info:
        load_tensors(path, params, torch.bfloat16, prefixes=spec.tensor_prefixes)
    err = info.value
    assert err.missing == ["text.blocks.1.ln.bias", "text.lm_head.bias"]
    assert err.unexpected == ["stray", "text.blocks.9.ln.weight"]
    assert len(err.mismatched) == 1 and "text.blocks.0.mlp.fc1.weight" in err.mismatched[0]
    text = str(err)
    assert "missing (2)" in text and "unexpected (2)" in text and "stored [8, 8], the model needs [256, 64]" in text


def test_loader_reads_pt_checkpoints_with_the_same_report(tmp_path):
    """A ``.pt`` file of tensors goes through the weights-only, memory-mapped loader
    (``kestrel/models/moondream/weights.py:560-566``) and the same checks as safetensors."""
    from kestrel_amd.weights.loader import find_weights

    spec, params = _params()
    stored = load_file(helpers.model_dir("A") + "/model.safetensors")
    good = {"model." + k.replace("text.blocks", "text._orig_mod.blocks"): v for k, v in stored.items()}
    torch.save(good, str(tmp_path / "model.pt"))
    assert find_weights(tmp_path, "model.safetensors") == tmp_path / "model.pt"
    got = load_tensors(tmp_path / "model.pt", params, torch.float32, prefixes=spec.tensor_prefixes)
    want = load_tensors(helpers.model_dir("A") + "/model.safetensors", params, torch.float32, prefixes=spec.tensor_prefixes)
    assert set(got) == set(want) and all(torch.equal(got[k], want[k]) for k in want)
    bad = dict(stored)
    del bad["text.lm_head.bias"]
    bad["text.wte"] = torch.zeros(5, 5)
    bad["stray"] = torch.zeros(1)
    torch.save(bad, str(tmp_path / "bad.pt"))
    with pytest.raises(WeightsError) as info:
        load_tensors(tmp_path / "bad.pt", params, torch.bfloat16, prefixes=spec.tensor_prefixes)
    assert info.value.missing == ["text.lm_head.bias"] and info.value.unexpected == ["stray"]
    assert "text.wte: stored [5, 5]" in info.value.mismatched[0]
    # a file that is not a mapping of tensors, and one that would have to run code to be read
    torch.save([1, 2, 3], str(tmp_path / "list.pt"))
    with pytest.raises(ValueError, match="mapping from tensor names"):
        load_tensors(tmp_path / "list.pt", params, torch.bfloat16)
    import pickle

    class Runs:
        def __reduce__(self):
            return (print, ("this must never be printed",))

    with open(tmp_path / "evil.pt", "wb") as handle:
        pickle.dump({"text.wte": Runs()}, handle)
    with pytest.raises(ValueError, match="weights-only loader"):
        load_tensors(tmp_path / "evil.pt", params, torch.bfloat16)
    with pytest.raises(FileNotFoundError, match="holds no weights"):
        find_weights(tmp_path / "nowhere", "model.safetensors")


def test_loader_refuses_integer_weights(tmp_path):
    spec, params = _params()
    stored = load_file(helpers.model_dir("A") + "/model.safetensors")
    stored["text.post_ln.bias"] = torch.zeros(64, dtype=torch.int32)
    path = tmp_path / "model.safetensors"
    save_file(stored, str(path))
    with pytest.raises(WeightsError, match="floating type"):
        load_tensors(path, params, torch.bfloat16, prefixes=spec.tensor_prefixes)


def test_missing_files(tmp_path):
    with pytest.raises(FileNotFoundError, match="config.json"):
        read_model_dir(tmp_path)
    (tmp_path / "config.json").write_text(json.dumps(helpers.TINY_A))
    spec, params = _params()
    with pytest.raises(FileNotFoundError):
        load_tensors(tmp_path / "model.safetensors", params, torch.float32)


def test_a_stale_library_that_cannot_be_rebuilt_is_an_error(tmp_path, monkeypatch):
    """A built library whose stamp does not match the sources must not run silently where there is
    no compiler: loading it is an error unless the environment says otherwise."""
    from kestrel_amd.csrc import build

    stale = tmp_path / "libka_core.so"
    stale.write_bytes(b"not a library")

    def no_compiler(name, verbose=True):
        raise build.KernelBuildError("hipcc not found")

    monkeypatch.setattr(build, "_find_built", lambda name: (stale, False))
    monkeypatch.setattr(build, "build", no_compiler)
    monkeypatch.setattr(build, "_loaded", {})
    monkeypatch.delenv("KESTREL_AMD_ALLOW_STALE", raising=False)
    with pytest.raises(build.KernelBuildError, match="older than its sources"):
        build.load("core")
    monkeypatch.setenv("KESTREL_AMD_ALLOW_STALE", "1")
    with pytest.raises(build.KernelBuildError, match="cannot load"):       # it is tried, and is no library
        build.load("core")
    monkeypatch.setattr(build, "_find_built", lambda name: (None, False))
    with pytest.raises(build.KernelBuildError, match="hipcc not found"):
        build.load("core")

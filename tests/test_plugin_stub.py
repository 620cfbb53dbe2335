"""The vLLM plugin mirror (quantexperiments_amd/vllm_ext/plugin.py) against a stand-in for the few vLLM names
it touches.  vLLM is not installed here, so this pins the plugin's own logic (config keys and environment
overrides, pickling, which method a layer gets, shape and tensor-parallel checks, the aux-section checks, and
on a GPU the create_weights -> apply / embedding path), not vLLM's behaviour."""

import os
import pickle
import sys
import types

import numpy as np
import pytest
import torch

from oracle import sq_oracle as O
from tests.helpers import rand_x, rel_max_err, synth


class _Current:
    model_dir = "."
    quant_config = None


def _install_stub():
    mods = {}

    def mod(name):
        m = types.ModuleType(name)
        mods[name] = m
        return m

    for n in ("vllm", "vllm.model_executor", "vllm.model_executor.layers", "vllm.model_executor.models"):
        mod(n).__path__ = []
    cfg = mod("vllm.config")

    def get_current_vllm_config():
        return types.SimpleNamespace(model_config=types.SimpleNamespace(model=_Current.model_dir, revision=None),
                                     quant_config=_Current.quant_config)
    cfg.get_current_vllm_config = get_current_vllm_config
    lin = mod("vllm.model_executor.layers.linear")
    lin.LinearBase = type("LinearBase", (torch.nn.Module,), {})
    lin.LinearMethodBase = type("LinearMethodBase", (), {})
    lin.UnquantizedLinearMethod = type("UnquantizedLinearMethod", (lin.LinearMethodBase,), {})
    q = mod("vllm.model_executor.layers.quantization")
    q.__path__ = []
    q.REGISTERED = {}

    def register_quantization_config(name):
        def deco(cls):
            q.REGISTERED[name] = cls
            return cls
        return deco
    q.register_quantization_config = register_quantization_config
    base = mod("vllm.model_executor.layers.quantization.base_config")
    base.QuantizeMethodBase = type("QuantizeMethodBase", (), {})
    base.QuantizationConfig = type("QuantizationConfig", (), {"__init__": lambda self: None})
    voc = mod("vllm.model_executor.layers.vocab_parallel_embedding")
    voc.VocabParallelEmbedding = type("VocabParallelEmbedding", (torch.nn.Module,), {})
    voc.ParallelLMHead = type("ParallelLMHead", (voc.VocabParallelEmbedding,), {})
    return mods


@pytest.fixture()
def plugin(monkeypatch):
    for k in list(os.environ):
        if k.startswith("SHAPEQUANT_"):
            monkeypatch.delenv(k)
    mods = _install_stub()
    for k, v in mods.items():
        monkeypatch.setitem(sys.modules, k, v)
    monkeypatch.delitem(sys.modules, "quantexperiments_amd.vllm_ext.plugin", raising=False)
    import importlib
    p = importlib.import_module("quantexperiments_amd.vllm_ext.plugin")
    p._embedding_is_ours = False
    yield p, mods
    sys.modules.pop("quantexperiments_amd.vllm_ext.plugin", None)


def _packed_dir(tmp_path, aux=True):
    """A model directory with a packed file: q/k/v of layer 0 (d = 4, K = 1024) + a 40 x 64 embedding / head."""
    from quantexperiments_amd import packed
    ss, entries = {}, {}
    for name, R in (("q_proj", 48), ("k_proj", 16), ("v_proj", 16)):
        s = synth(R, 64, 4, 10, seed=R)
        t, meta = packed.pack_tensors(torch.from_numpy(s.tags), torch.from_numpy(s.table), torch.from_numpy(s.row_scale),
                                      d=4, K=1024, G=1, M=1, seed=1)
        entries[f"model.layers.0.self_attn.{name}"] = (t, meta)
        ss[name] = s
    g = torch.Generator().manual_seed(3)
    w = (torch.randn(40, 64, generator=g) * 0.05)
    a = None
    if aux:
        eq, es = packed.q4_embed_pack(w)
        hq, hs, _ = packed.q8_pack(w)
        a = ({"aux.embed.q": eq, "aux.embed.scale": es, "aux.lm_head.q": hq, "aux.lm_head.scale": hs},
             {"embed": "q4_b32", "lm_head": "q8_b32", "dense": [], "config": {}, "vocab": 40, "hidden": 64, "tied": False})
    packed.save(tmp_path / "shapequant.packed", entries, base_model="t", aux=a)
    _Current.model_dir = str(tmp_path)
    return ss, w.numpy()


def test_config_keys_env_overrides_and_pickling(plugin, tmp_path, monkeypatch):
    p, mods = plugin
    assert mods["vllm.model_executor.layers.quantization"].REGISTERED["shapequant"] is p.ShapeQuantConfig
    c = p.ShapeQuantConfig.from_config({"packed_file": "shapequant.packed", "bmax": 16, "large": "chunked", "chunk_mb": 8})
    assert (c.packed_file, c.bmax, c.large, c.chunk_mb, c.embed_head, c.tune) == ("shapequant.packed", 16, "chunked", 8, "bf16", False)
    assert p.ShapeQuantConfig.get_name() == "shapequant" and p.ShapeQuantConfig.get_min_capability() == 0
    assert p.ShapeQuantConfig.get_supported_act_dtypes() == [torch.bfloat16, torch.float16]
    assert p.ShapeQuantConfig.get_config_filenames() == []
    with pytest.raises(KeyError):
        p.ShapeQuantConfig.from_config({})
    with pytest.raises(ValueError, match="bf16 | packed"):
        p.ShapeQuantConfig("f", embed_head="q4")
    monkeypatch.setenv("SHAPEQUANT_LARGE", "dequant")
    monkeypatch.setenv("SHAPEQUANT_BMAX", "64")
    monkeypatch.setenv("SHAPEQUANT_TUNE", "1")
    c2 = p.ShapeQuantConfig("f", large="fused", bmax=8)
    assert c2.large == "dequant" and c2.bmax == 32 and c2.tune          # the kernels take at most 32 rows
    _packed_dir(tmp_path)
    assert c.pf.meta and c._pf is not None
    c3 = pickle.loads(pickle.dumps(c))                                  # the open file does not travel
    assert c3._pf is None and c3.packed_file == c.packed_file and c3.large == "chunked"
    assert "shapequant.packed" in repr(c3)
    with pytest.raises(FileNotFoundError):
        _Current.model_dir = "not-a-directory"
        p.ShapeQuantConfig("nowhere.packed").pf


def test_which_method_a_layer_gets(plugin, tmp_path):
    p, mods = plugin
    _packed_dir(tmp_path)
    lin = mods["vllm.model_executor.layers.linear"]
    voc = mods["vllm.model_executor.layers.vocab_parallel_embedding"]
    c = p.ShapeQuantConfig("shapequant.packed")
    assert c.get_quant_method(torch.nn.LayerNorm(4), "model.norm") is None
    m = c.get_quant_method(lin.LinearBase(), "model.layers.0.self_attn.qkv_proj")
    assert isinstance(m, p.ShapeQuantLinearMethod)
    assert m.pieces == [f"model.layers.0.self_attn.{n}" for n in ("q_proj", "k_proj", "v_proj")]
    assert isinstance(c.get_quant_method(lin.LinearBase(), "model.layers.0.mlp.down_proj"), lin.UnquantizedLinearMethod)
    assert isinstance(c.get_quant_method(lin.LinearBase(), "mtp.layers.0.self_attn.qkv_proj"), lin.UnquantizedLinearMethod)
    assert c.get_quant_method(voc.ParallelLMHead(), "lm_head") is None
    assert c.get_quant_method(voc.VocabParallelEmbedding(), "model.embed_tokens") is None
    cp = p.ShapeQuantConfig("shapequant.packed", embed_head="packed")
    assert cp.get_quant_method(voc.ParallelLMHead(), "lm_head").what == "lm_head"
    assert cp.get_quant_method(voc.VocabParallelEmbedding(), "model.embed_tokens").what == "embed"
    # tensor parallelism is refused before anything touches the GPU
    with pytest.raises(NotImplementedError, match="tensor parallelism"):
        m.create_weights(lin.LinearBase(), 32, [80], 64, 80, torch.bfloat16)
    with pytest.raises(NotImplementedError, match="tensor parallelism"):
        m.create_weights(lin.LinearBase(), 64, [40], 64, 80, torch.bfloat16)
    with pytest.raises(NotImplementedError, match="tensor parallelism"):
        p.ShapeQuantAuxMethod(cp, "lm_head").create_weights(voc.ParallelLMHead(), 64, [20], 64, 40, torch.bfloat16)


def test_aux_checks_and_head_keep(plugin, tmp_path, monkeypatch):
    p, mods = plugin
    voc = mods["vllm.model_executor.layers.vocab_parallel_embedding"]
    _packed_dir(tmp_path, aux=False)
    c = p.ShapeQuantConfig("shapequant.packed", embed_head="packed")
    with pytest.raises(ValueError, match="lm_head is None"):
        p.ShapeQuantAuxMethod(c, "lm_head").create_weights(voc.ParallelLMHead(), 64, [40], 64, 40, torch.bfloat16)
    _packed_dir(tmp_path, aux=True)
    c = p.ShapeQuantConfig("shapequant.packed", embed_head="packed")
    with pytest.raises(ValueError, match=r"\[40, 64\], layer is \[32, 64\]"):        # fewer rows than the file
        p._check_aux(c, "embed", 32, 64)
    with pytest.raises(ValueError, match="layer is"):
        p._check_aux(c, "lm_head", 48, 128)
    p._check_aux(c, "lm_head", 48, 64)                                               # a padded vocabulary is fine
    with pytest.raises(RuntimeError, match="token embedding was not built"):         # head before embedding
        p.ShapeQuantAuxMethod(c, "lm_head").create_weights(voc.ParallelLMHead(), 64, [48], 64, 48, torch.bfloat16)
    with pytest.raises(RuntimeError):
        p.ShapeQuantAuxMethod(c, "lm_head").embedding(voc.ParallelLMHead(), torch.zeros(1, dtype=torch.long))
    with pytest.raises(RuntimeError):
        p.ShapeQuantAuxMethod(c, "embed").apply(voc.VocabParallelEmbedding(), torch.zeros(1, 64))
    assert p._kept_token_ids() is None
    np.save(tmp_path / "keep.npy", np.array([0, 3, 2], np.int64))
    monkeypatch.setenv("SHAPEQUANT_HEAD_KEEP", "keep.npy")                           # relative: in the model directory
    with pytest.raises(ValueError, match="ascending"):
        p._kept_token_ids()
    np.save(tmp_path / "keep.npy", np.array([0, 2, 39], np.int64))
    assert p._kept_token_ids().tolist() == [0, 2, 39]


@pytest.mark.gpu
def test_create_weights_apply_and_embedding_on_the_gpu(plugin, tmp_path, monkeypatch):
    p, mods = plugin
    lin = mods["vllm.model_executor.layers.linear"]
    voc = mods["vllm.model_executor.layers.vocab_parallel_embedding"]
    ss, w = _packed_dir(tmp_path)
    c = p.ShapeQuantConfig("shapequant.packed", embed_head="packed")
    layer = lin.LinearBase()
    m = c.get_quant_method(layer, "model.layers.0.self_attn.qkv_proj")
    with pytest.raises(ValueError, match="vLLM layer is"):
        m.create_weights(lin.LinearBase(), 64, [96], 64, 96, torch.bfloat16)
    m.create_weights(layer, 64, [48, 16, 16], 64, 80, torch.bfloat16)
    m.process_weights_after_loading(layer)
    x = rand_x(5, 64, torch.bfloat16, seed=1)
    bias = torch.arange(80, dtype=torch.bfloat16).cuda()
    y = m.apply(layer, x.cuda())
    ref = np.concatenate([O.linear(x.float().numpy(), ss[n].decode()) for n in ("q_proj", "k_proj", "v_proj")], axis=1)
    assert y.shape == (5, 80) and y.dtype == torch.bfloat16
    assert rel_max_err(y.float().cpu().numpy(), ref) < 2.0 ** -7
    assert torch.equal(m.apply(layer, x.cuda(), bias), y + bias)
    # embedding, then head (padded to 48 rows), both behind their ops
    emb_layer, head_layer = voc.VocabParallelEmbedding(), voc.ParallelLMHead()
    em, hm = c.get_quant_method(emb_layer, "model.embed_tokens"), c.get_quant_method(head_layer, "lm_head")
    em.create_weights(emb_layer, 64, [48], 64, 48, torch.bfloat16)
    hm.create_weights(head_layer, 64, [48], 64, 48, torch.bfloat16)
    ids = torch.tensor([[0, 39, 7]]).cuda()
    e = em.embedding(emb_layer, ids)
    eq, es = O.q4_embed_pack(w)
    assert e.shape == (1, 3, 64) and np.array_equal(e.float().cpu().numpy().reshape(3, 64), O.round_bf16(O.q4_embed_rows(eq, es, [0, 39, 7])))
    logits = hm.apply(head_layer, e.view(3, 64))
    hq, hs, _ = O.q8_pack(w)
    ref = O.q8_linear(e.view(3, 64).float().cpu().numpy(), hq, hs)
    assert logits.shape == (3, 48) and rel_max_err(logits[:, :40].float().cpu().numpy(), ref) < 2.0 ** -7 and not logits[:, 40:].any()
    # a pruned head: SHAPEQUANT_HEAD_KEEP
    np.save(tmp_path / "keep.npy", np.array([1, 5, 39], np.int64))
    monkeypatch.setenv("SHAPEQUANT_HEAD_KEEP", str(tmp_path / "keep.npy"))
    pruned = voc.ParallelLMHead()
    hm.create_weights(pruned, 64, [48], 64, 48, torch.bfloat16)
    lp = hm.apply(pruned, e.view(3, 64)).float().cpu()
    assert rel_max_err(lp[:, [1, 5, 39]].numpy(), ref[:, [1, 5, 39]]) < 2.0 ** -7
    assert torch.isinf(lp[:, 0]).all() and torch.isinf(lp[:, 47]).all()
    # the table in pinned host memory
    monkeypatch.setenv("SHAPEQUANT_EMBED_HOST", "1")
    host_layer = voc.VocabParallelEmbedding()
    em.create_weights(host_layer, 64, [48], 64, 48, torch.bfloat16)
    assert host_layer.sq_shards.q.device.type == "cpu" and torch.equal(em.embedding(host_layer, ids), e)

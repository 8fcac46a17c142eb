"""The branches of the patch layer that run when SGLang and vLLM are importable
(``patch_model_runner``, ``patch_input_metadata``, ``patch_model``): module trees with
the attributes the reference touches are put into ``sys.modules`` and the same
attributes must come out overwritten (tr.py:452-472, 475-655, 658-699, 868-882)."""

import enum
import sys
import types

import pytest
import torch

from tokenselect_amd.patcher import token_retrieval as tr


class _ForwardMode(enum.Enum):
    PREFILL = 1
    EXTEND = 2
    DECODE = 3


class _BaseRunner:
    def __init__(self, **kwargs):
        self.__dict__.update(kwargs)
        self.base_init_ran = True


class _BaseMeta:
    def __init__(self, **kwargs):
        self.kwargs = dict(kwargs)
        self.__dict__.update(kwargs)
        self.calls = []

    def compute_positions(self, batch):
        self.calls.append("compute_positions")

    def compute_extend_infos(self, batch):
        self.calls.append("compute_extend_infos")

    def init_multimuldal_info(self, batch):
        self.calls.append("init_multimuldal_info")


class _Loader:
    def load_model(self, **kwargs):
        return kwargs["model"]


def _module(name, **attrs):
    m = types.ModuleType(name)
    m.__dict__.update(attrs)
    return m


@pytest.fixture
def frameworks(monkeypatch):
    """sglang.srt.model_executor.{model_runner, forward_batch_info} and
    vllm.model_executor.{layers.rotary_embedding, model_loader.loader}."""
    original_update = lambda *a, **k: "flashinfer plan"  # noqa: E731
    mods = {
        "sglang": _module("sglang"),
        "sglang.srt": _module("sglang.srt"),
        "sglang.srt.model_executor": _module("sglang.srt.model_executor"),
        "sglang.srt.model_executor.model_runner": _module(
            "sglang.srt.model_executor.model_runner", ModelRunner=_BaseRunner),
        "sglang.srt.model_executor.forward_batch_info": _module(
            "sglang.srt.model_executor.forward_batch_info", InputMetadata=_BaseMeta,
            ForwardMode=_ForwardMode, update_flashinfer_indices=original_update),
        "vllm": _module("vllm"),
        "vllm.model_executor": _module("vllm.model_executor"),
        "vllm.model_executor.layers": _module("vllm.model_executor.layers"),
        "vllm.model_executor.layers.rotary_embedding": _module(
            "vllm.model_executor.layers.rotary_embedding", get_rope=lambda *a, **k: "a rope module"),
        "vllm.model_executor.model_loader": _module("vllm.model_executor.model_loader"),
        "vllm.model_executor.model_loader.loader": _module(
            "vllm.model_executor.model_loader.loader", DefaultModelLoader=_Loader),
    }
    for name, mod in mods.items():
        monkeypatch.setitem(sys.modules, name, mod)
        if "." in name:
            parent, child = name.rsplit(".", 1)
            monkeypatch.setattr(mods[parent], child, mod, raising=False)
    monkeypatch.setattr(_Loader, "load_model", _Loader.load_model)   # restored after the test
    return mods


class _ModelConfig:
    num_hidden_layers, head_dim, num_attention_heads = 32, 128, 32

    def get_num_kv_heads(self, tp_size):
        return 8 // tp_size


def test_model_runner_is_replaced_and_builds_the_retriever(frameworks, monkeypatch):
    built = {}

    class Recorder:
        def __init__(self, *args):
            built["args"] = args

    monkeypatch.setattr(tr, "ReqToTokenRetriever", Recorder)
    tr.patch(rope_base=5e5, max_n_tokens=1048576, top_k=2048, n_init=128, n_local=512)
    runner_mod = frameworks["sglang.srt.model_executor.model_runner"]
    patched = runner_mod.ModelRunner                     # tr.py:472
    assert patched is not _BaseRunner and issubclass(patched, _BaseRunner)
    pool = object()
    runner = patched(model_config=_ModelConfig(), tp_size=2, token_to_kv_pool=pool,
                     dtype=torch.bfloat16, max_total_num_tokens=12345)
    assert runner.base_init_ran
    assert isinstance(runner.req_to_token_retriever, Recorder)
    # tr.py:456-468: layers, head_dim, heads, kv heads of the rank, fingerprint dim, table
    # capacity, the pool (aliased), dtype, device
    assert built["args"] == (32, 128, 32, 4, 4 * 128, 1048576, pool, torch.bfloat16, "cuda")


class _Retrievers:
    def __init__(self):
        self.asked = []

    def get_token_retriever(self, rid):
        self.asked.append(rid)
        return f"retriever of {rid}"


def _batch(rid="req-7"):
    return types.SimpleNamespace(
        batch_size=lambda: 1, req_pool_indices=torch.tensor([3]), seq_lens=torch.tensor([700]),
        reqs=[types.SimpleNamespace(rid=rid, prefix_indices=[])], out_cache_loc=torch.tensor([9]),
        return_logprob=False, top_logprobs_nums=[0])


def test_input_metadata_carries_the_running_requests_retriever(frameworks):
    tr.patch()
    fbi = frameworks["sglang.srt.model_executor.forward_batch_info"]
    meta_cls = fbi.InputMetadata                         # tr.py:652
    assert meta_cls is not _BaseMeta and issubclass(meta_cls, _BaseMeta)
    runner = types.SimpleNamespace(req_to_token_pool="r2t", token_to_kv_pool="kv",
                                   req_to_token_retriever=_Retrievers(), sliding_window_size=None)
    batch = _batch()
    meta = meta_cls.from_schedule_batch(runner, batch, _ForwardMode.DECODE)
    assert runner.req_to_token_retriever.asked == ["req-7"]          # tr.py:524-526
    assert meta.token_retriever == "retriever of req-7"
    # the keyword list of tr.py:517-531, minus token_retriever, which the subclass pops
    assert set(meta.kwargs) == {"forward_mode", "batch_size", "req_pool_indices", "seq_lens",
                                "req_to_token_pool", "token_to_kv_pool", "out_cache_loc",
                                "return_logprob", "top_logprobs_nums"}
    assert meta.req_to_token_pool == "r2t" and meta.token_to_kv_pool == "kv" and meta.batch_size == 1
    assert meta.calls == ["compute_positions", "compute_extend_infos"]
    assert not hasattr(meta, "total_num_tokens") and meta.flashinfer_use_ragged is False
    extend = meta_cls.from_schedule_batch(runner, batch, _ForwardMode.EXTEND)
    assert extend.total_num_tokens == 700                             # tr.py:537-542
    assert extend.calls == ["compute_positions", "compute_extend_infos", "init_multimuldal_info"]
    assert extend.flashinfer_use_ragged is False                      # tr.py:492


def test_flashinfer_index_planning_is_replaced_by_a_function_that_plans_nothing(frameworks):
    tr.patch()
    fbi = frameworks["sglang.srt.model_executor.forward_batch_info"]
    update = fbi.update_flashinfer_indices                # tr.py:653-655
    assert update is tr.patched_forward_batch_info_update_flashinfer_indices
    runner = types.SimpleNamespace(sliding_window_size=None)
    assert update(_ForwardMode.DECODE, runner, torch.tensor([0]), torch.tensor([5]), None) is None
    with pytest.raises(NotImplementedError, match="Ragged"):          # tr.py:589
        update(_ForwardMode.EXTEND, runner, torch.tensor([0]), torch.tensor([5]), torch.tensor([0]),
               flashinfer_use_ragged=True)
    runner.sliding_window_size = 4096
    with pytest.raises(NotImplementedError, match="Sliding window"):  # tr.py:650
        update(_ForwardMode.DECODE, runner, torch.tensor([0]), torch.tensor([5]), None)


def test_loader_and_rope_factory_are_wrapped(frameworks):
    class Attn:            # the model's attention module and its RadixAttention
        pass

    class Radix:
        pass

    def layer():
        a = Attn()
        a.attn = Radix()
        return types.SimpleNamespace(self_attn=a)

    model = types.SimpleNamespace(model=types.SimpleNamespace(layers=[layer(), layer()]))
    tr.patch()
    rope = frameworks["vllm.model_executor.layers.rotary_embedding"]
    assert rope.get_rope("anything", base=1e6) is None   # tr.py:878-882: K stays un-rotated
    loaded = _Loader().load_model(model=model)           # tr.py:661-699 through patch_attention
    assert loaded is model
    assert Attn.forward is tr.patched_meta_attention_forward            # tr.py:868-875
    assert Radix.forward is tr.patched_radix_attention_forward
    assert Radix.store_kv_cache is tr.patched_radix_attention_store_kv_cache

"""The two model-runner hooks of the plugin contract that touch the attention path, driven through a fake runner
(the reference pins them in tests/unit/platform/test_npu_model_runner.py:96-218): get_kv_cache_spec publishes
MLAAttentionSpec(head_size = 576 + index_head_dim) for DSA models, _reshape_kv_cache_tensors hands every layer's raw
allocation to its backend's reshape_kv_cache with the spec's geometry."""
from types import SimpleNamespace

import pytest
import torch

from omni_npu_amd._vllm_compat import AttentionSpec, MLAAttentionSpec
from omni_npu_amd.attention.backends.dsa import NPUDSABackend
from omni_npu_amd.attention.backends.mla import NPUMLABackend
from omni_npu_amd.worker.hip_worker import KVCacheHooksMixin, kv_cache_dtype_and_head_size


class _BaseRunner:
    def get_kv_cache_spec(self):
        return {"not_mla": "stock spec"}


class FakeRunner(KVCacheHooksMixin, _BaseRunner):
    def __init__(self, use_mla=True, hf_config=None, cache_dtype="auto", block_size=128, dtype=torch.bfloat16, layers=None):
        self.vllm_config = SimpleNamespace(
            model_config=SimpleNamespace(use_mla=use_mla, hf_config=hf_config or SimpleNamespace(), dtype=dtype),
            cache_config=SimpleNamespace(block_size=block_size, cache_dtype=cache_dtype))
        self._layers = layers or {"layer_0": SimpleNamespace(head_size=576), "layer_1": SimpleNamespace(head_size=576)}
        self.runner_only_attn_layers = set()
        self._groups = []

    def _attention_layers(self):
        return self._layers

    def _kv_cache_spec_attn_group_iterator(self):
        return self._groups


def test_get_kv_cache_spec_mla_bf16():
    specs = FakeRunner().get_kv_cache_spec()
    assert set(specs) == {"layer_0", "layer_1"}
    for spec in specs.values():
        assert isinstance(spec, MLAAttentionSpec)
        assert (spec.block_size, spec.num_kv_heads, spec.head_size, spec.dtype, spec.cache_dtype_str) == \
            (128, 1, 576, torch.bfloat16, "auto")
        assert spec.page_size_bytes == 128 * 576 * 2


def test_get_kv_cache_spec_dsa_adds_the_indexer_keys():
    """Reference: head_size = attn.head_size + index_head_dim when the model has index_topk (npu_model_runner.py:171-187)."""
    hf = SimpleNamespace(index_topk=2048, index_head_dim=128)
    layers = {"a": SimpleNamespace(head_size=576), "b": SimpleNamespace(head_size=32)}
    specs = FakeRunner(hf_config=hf, block_size=16, dtype=torch.float16, layers=layers).get_kv_cache_spec()
    assert set(specs) == set(layers)
    for name, spec in specs.items():
        assert isinstance(spec, MLAAttentionSpec)
        assert spec.head_size == layers[name].head_size + 128 and spec.block_size == 16 and spec.num_kv_heads == 1
        assert spec.dtype == torch.float16 and spec.cache_dtype_str == "auto"
    # a model with index_topk but no index_head_dim gets the default width
    specs = FakeRunner(hf_config=SimpleNamespace(index_topk=4)).get_kv_cache_spec()
    assert all(s.head_size == 576 + 128 for s in specs.values())


def test_get_kv_cache_spec_fp8_row_and_fp8_dsa_refusal():
    specs = FakeRunner(cache_dtype="fp8").get_kv_cache_spec()
    for spec in specs.values():
        assert (spec.dtype, spec.head_size, spec.cache_dtype_str) == (torch.uint8, 656, "fp8")
        assert spec.page_size_bytes == 128 * 656
    assert kv_cache_dtype_and_head_size("fp8_e4m3", torch.bfloat16, 576) == (torch.uint8, 656)
    assert kv_cache_dtype_and_head_size("auto", torch.bfloat16, 576, 128) == (torch.bfloat16, 704)
    with pytest.raises(NotImplementedError, match="DSA"):
        FakeRunner(cache_dtype="fp8", hf_config=SimpleNamespace(index_topk=2048, index_head_dim=128)).get_kv_cache_spec()


def test_get_kv_cache_spec_without_mla_defers_to_the_stock_runner():
    assert FakeRunner(use_mla=False).get_kv_cache_spec() == {"not_mla": "stock spec"}


def test_reshape_kv_cache_tensors_calls_the_backend_with_the_spec_geometry():
    """Mirrors the reference test: a recording backend, one layer, 2048 raw bytes of an (2, 1, 4, fp16) spec = 64 blocks."""
    spec = AttentionSpec(block_size=2, num_kv_heads=1, head_size=4, dtype=torch.float16)
    seen = {}

    class RecordingBackend:
        @staticmethod
        def reshape_kv_cache(raw_tensor, num_blocks, block_size, num_kv_heads, head_size, dtype):
            seen["args"] = (raw_tensor, num_blocks, block_size, num_kv_heads, head_size, dtype)
            return torch.ones(3, 3, dtype=dtype)

    runner = FakeRunner()
    raw = torch.zeros(2048, dtype=torch.uint8)
    runner._groups = [SimpleNamespace(kv_cache_spec=spec, backend=RecordingBackend, layer_names=["layer_0", "skipped"])]
    runner.runner_only_attn_layers = {"skipped"}
    out = runner._reshape_kv_cache_tensors(kv_cache_config=object(), kv_cache_raw_tensors={"layer_0": raw, "skipped": raw},
                                           kernel_block_sizes=[2])
    assert seen["args"][0] is raw and seen["args"][1:] == (64, 2, 1, 4, torch.float16)
    assert set(out) == {"layer_0"} and torch.equal(out["layer_0"], torch.ones(3, 3, dtype=torch.float16))


def test_reshape_kv_cache_tensors_with_the_real_backends():
    """MLA: two tensors; DSA (704 wide): three, the third holding the indexer keys; a raw size that is not a whole number
    of pages is refused."""
    runner = FakeRunner()
    mla_spec = MLAAttentionSpec(block_size=128, num_kv_heads=1, head_size=576, dtype=torch.bfloat16)
    dsa_spec = MLAAttentionSpec(block_size=128, num_kv_heads=1, head_size=704, dtype=torch.bfloat16)
    raws = {"m": torch.zeros(3 * mla_spec.page_size_bytes, dtype=torch.uint8),
            "d": torch.zeros(2 * dsa_spec.page_size_bytes, dtype=torch.uint8)}
    runner._groups = [SimpleNamespace(kv_cache_spec=mla_spec, backend=NPUMLABackend, layer_names=["m"]),
                      SimpleNamespace(kv_cache_spec=dsa_spec, backend=NPUDSABackend, layer_names=["d"])]
    out = runner._reshape_kv_cache_tensors(None, raws)
    assert [tuple(x.shape) for x in out["m"]] == [(3, 128, 512), (3, 128, 64)]
    assert [tuple(x.shape) for x in out["d"]] == [(2, 128, 1, 512), (2, 128, 1, 64), (2, 128, 1, 128)]
    assert all(x.dtype == torch.bfloat16 for x in out["m"] + out["d"])
    assert out["m"][0].data_ptr() == raws["m"].data_ptr()          # views of the raw allocation, not copies
    runner._groups = [SimpleNamespace(kv_cache_spec=mla_spec, backend=NPUMLABackend, layer_names=["m"])]
    with pytest.raises(AssertionError):
        runner._reshape_kv_cache_tensors(None, {"m": torch.zeros(mla_spec.page_size_bytes + 2, dtype=torch.uint8)})


def test_dsa_impl_refuses_an_fp8_cache():
    from omni_npu_amd.attention.backends.dsa import NPUDSAImpl
    with pytest.raises(NotImplementedError, match="fp8"):
        NPUDSAImpl(num_heads=16, head_size=576, scale=0.1, num_kv_heads=1, alibi_slopes=None, sliding_window=None,
                   kv_cache_dtype="fp8", logits_soft_cap=None, attn_type="decoder", kv_sharing_target_layer_name=None,
                   q_lora_rank=None, kv_lora_rank=512, qk_nope_head_dim=128, qk_rope_head_dim=64, qk_head_dim=192,
                   v_head_dim=128, kv_b_proj=None, indexer=None)

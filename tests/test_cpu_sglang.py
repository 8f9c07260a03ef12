"""SGLang plugin mirror, host logic only: the routing-order known answer of the reference's
tests/test_sglang.py:19-39 (data vectors of that test), the environment contract and the hook
registration of camblas/sglang.py:199-222 against a stand-in for SGLang's hook registry."""

import sys
import types

import pytest
import torch

from camblas_amd import sglang as plugin


def test_canonical_prefill_routing_known_answer():
    routed = torch.tensor([2, 0, 1, 2, 1, 0, 2, 2])
    ids = torch.tensor([5, 8, 1, 8, 4, 8, 8, 2, 7, 0, 6, 3, 123, -8, 43, 0])
    experts = torch.tensor([0, 1, 2, -1])
    original = ids.clone()
    count = torch.tensor([12])
    expected = torch.tensor([1, 5, 8, 8, 2, 4, 8, 8, 0, 3, 6, 7, 8, 8, 8, 8])
    actual = plugin.canonical_moe_tokens(ids, experts, count, 4, routed.numel())
    assert torch.equal(actual, expected)
    assert torch.equal(ids, original)
    valid = actual < routed.numel()
    assert torch.equal(routed[actual[valid]], experts.repeat_interleave(4)[valid])
    # another valid alignment of the same routing gives the same order
    alternate = ids[torch.tensor([2, 0, 3, 1, 7, 4, 5, 6, 11, 10, 8, 9, 15, 14, 13, 12])]
    assert torch.equal(plugin.canonical_moe_tokens(alternate, experts, count, 4, 8), expected)
    assert actual.dtype == ids.dtype


def test_canonical_routing_brute_force():
    # every live block ends up sorted, keeps its multiset of entries, and dead capacity is padding
    generator = torch.Generator().manual_seed(5)
    for _ in range(20):
        blocks, size, choices = 6, 4, 40
        live_blocks = int(torch.randint(1, blocks + 1, (1,), generator=generator))
        ids = torch.randint(0, choices + 1, (blocks * size,), generator=generator, dtype=torch.int32)
        experts = torch.randperm(blocks, generator=generator).sort().values
        count = torch.tensor([live_blocks * size])
        got = plugin.canonical_moe_tokens(ids, experts, count, size, choices)
        for block in range(blocks):
            mine, theirs = got[block * size:(block + 1) * size], ids[block * size:(block + 1) * size]
            if block < live_blocks:
                assert torch.equal(mine, theirs.sort().values)
            else:
                assert (mine == choices).all()


def test_operation_selection():
    assert plugin.selected_operations({}) == set()
    assert plugin.selected_operations({"CAMBLAS_SGLANG_OPS": "linear,,fp8"}) == {"linear", "fp8"}
    with pytest.raises(ValueError, match="Unknown CAMBLAS SGLang operations"):
        plugin.selected_operations({"CAMBLAS_SGLANG_OPS": "linear,int4"})


@pytest.fixture
def registry(monkeypatch):
    """Minimal double of sglang.srt.plugins.hook_registry: records what install() registers."""
    recorded = []
    module = types.ModuleType("sglang.srt.plugins.hook_registry")

    class HookType:
        AROUND = "around"

    class HookRegistry:
        @staticmethod
        def register(target, function, kind):
            recorded.append((target, function, kind))

    module.HookType, module.HookRegistry = HookType, HookRegistry
    for name in ("sglang", "sglang.srt", "sglang.srt.plugins"):
        monkeypatch.setitem(sys.modules, name, types.ModuleType(name))
    monkeypatch.setitem(sys.modules, "sglang.srt.plugins.hook_registry", module)
    for name in ("CAMBLAS_SGLANG_OPS", "CAMBLAS_SGLANG_STABLE_MOE", "CAMBLAS_SGLANG_ALGORITHM"):
        monkeypatch.delenv(name, raising=False)
    return recorded


def test_install_registers_nothing_by_default(registry):
    plugin.install()
    assert registry == []


def test_install_registers_the_reference_hook_targets(registry, monkeypatch):
    monkeypatch.setenv("CAMBLAS_SGLANG_STABLE_MOE", "1")
    plugin.install()
    assert [(t, k) for t, _, k in registry] == [(plugin.MOE_ALIGN_TARGET, "around")]
    del registry[:]
    monkeypatch.delenv("CAMBLAS_SGLANG_STABLE_MOE")
    monkeypatch.setenv("CAMBLAS_SGLANG_OPS", "linear,fp8")
    monkeypatch.setattr(plugin, "build_hooks", lambda selected: {name: (lambda original, *a: original(*a))
                                                                 for name in sorted(selected)})
    from camblas_amd import _kernels

    chosen, installed = [], []
    monkeypatch.setattr(_kernels, "set_algorithm", chosen.append)
    # "linear" also routes torch.mm / addmm / F.linear through the library (ref: camblas/sglang.py:245-248)
    from camblas_amd import _native
    import types

    monkeypatch.setattr(_native, "tensor_module",
                        lambda: types.SimpleNamespace(install_torch_backend=installed.append))
    plugin.install()
    assert [t for t, _, _ in registry] == ["fp8", "linear"] and chosen == ["auto"]
    assert installed == [_native.ALGORITHMS["auto"]]
    monkeypatch.setenv("CAMBLAS_SGLANG_OPS", "fp8")
    plugin.install()
    assert installed == [_native.ALGORITHMS["auto"]]  # not without "linear"
    monkeypatch.setenv("CAMBLAS_SGLANG_OPS", "bmm")
    with pytest.raises(ValueError):
        plugin.install()


def test_hook_targets_are_the_reference_ones():
    # ref: camblas/sglang.py:287-291, :540-544, :641-645, :742-746, :192-196
    assert plugin.LINEAR_TARGET.endswith("UnquantizedLinearMethod.apply")
    assert plugin.BATCHED_LINEAR_TARGET == "sglang.srt.layers.linear.ColumnParallelBatchedLinear.forward"
    assert plugin.FP8_BLOCK128_TARGET.endswith("deepgemm_w8a8_block_fp8_linear_with_fallback")
    assert plugin.FP8_BLOCK32_PRODUCT_TARGET.endswith("w8a8_block_fp8_matmul_triton")
    assert plugin.FP8_BLOCK32_LINEAR_TARGET.endswith("triton_w8a8_block_fp8_linear")
    assert plugin.MOE_ALIGN_TARGET.endswith("moe_align_block_size.moe_align_block_size")
    # ref: camblas/sglang.py:452-456
    assert plugin.FP8_MOE_TARGET == "sglang.srt.layers.moe.moe_runner.triton_utils.fused_moe.fused_experts"


def test_stable_moe_hook_only_reorders_prefill():
    ids = torch.tensor([3, 1, 2, 0, 9, 9, 9, 9], dtype=torch.int32)
    experts = torch.tensor([0, -1])
    count = torch.tensor([4])

    def original(topk_ids, block_size, num_experts):
        return ids.clone(), experts, count

    decode = plugin.stable_moe_hook(original, torch.zeros((1, 4), dtype=torch.int32), 4, 1)
    assert torch.equal(decode[0], ids)
    prefill = plugin.stable_moe_hook(original, torch.zeros((2, 2), dtype=torch.int32), 4, 1)
    assert torch.equal(prefill[0], torch.tensor([0, 1, 2, 3, 4, 4, 4, 4], dtype=torch.int32))

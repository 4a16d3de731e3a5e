"""CPU-side checks: the C-ABI library loads and exports every symbol the header declares, the host
mirror of the reference interface behaves like the reference for argument handling, and nothing in
the package reaches into the checker."""
import ctypes
import json
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
KATS = json.load(open(os.path.join(ROOT, "tests", "golden", "reference_kats.json")))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "moe355.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(moe355_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from vllm_ascend_amd import _lib

    lib = ctypes.CDLL(_lib.LIB_PATH)
    names = _declared_symbols()
    assert len(names) >= 15
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in include/moe355.h but not exported"
    # the ctypes prototypes cover the same set
    assert sorted(_lib.PROTOTYPES) == names


def test_abi_version_and_strerror():
    from vllm_ascend_amd import _lib

    lib = _lib.load()
    assert lib.moe355_abi_version() == _lib.ABI_VERSION
    assert lib.moe355_strerror(0) == b"ok"
    assert b"workspace" in lib.moe355_strerror(-3)


def test_argument_validation_without_gpu():
    """Rejections happen on the host before any launch, so they can be exercised without a GPU."""
    from vllm_ascend_amd import _lib

    lib = _lib.load()
    one = ctypes.c_void_p(256)  # never dereferenced: every call below is refused first
    assert lib.moe355_dynamic_quant(one, 1, -1, 8, one, one, None) == -1
    assert lib.moe355_dynamic_quant(one, 0, 4, 8, one, one, None) == -5  # fp32 input not supported
    assert lib.moe355_gating_top_k(one, 0, None, 4, 4096, 8, 1, 1, 1, 1, 0, 0, 1.0, 1e-20, one, one, None, None, 0,
                                   None) == -2  # E > 2048
    assert lib.moe355_gating_top_k(one, 0, None, 4, 64, 8, 1, 3, 1, 1, 0, 0, 1.0, 1e-20, one, one, None, None, 0,
                                   None) == -2  # E % group_count
    assert lib.moe355_gating_top_k(one, 0, None, 4, 64, 8, 1, 1, 1, 1, 2, 0, 1.0, 1e-20, one, one, None, None, 0,
                                   None) == -1  # norm_type
    assert lib.moe355_gmm_i32(one, one, one, 0, 4, 48, 64, 2, one, one, 256, None) == -2  # K % 32
    assert lib.moe355_gmm_i32(one, one, one, 7, 4, 64, 64, 2, one, one, 256, None) == -1  # group list type
    assert lib.moe355_gmm1_swiglu_quant(one, one, one, one, one, 0, 4, 64, 64, 2, 0.0, one, one, None, 0,
                                        None) == -3  # no workspace
    assert lib.moe355_init_routing(one, 1, 4, 64, one, 2, 8, 5, 1, one, one, one, one, one, 1 << 20, None) == -5
    assert lib.moe355_format_cast_nz(one, 0, 2, 48, 64, one, None) == -2
    assert lib.moe355_token_unpermute(one, 0, one, one, 4, 2, 64, 8, None, one, None) == -5
    assert lib.moe355_init_routing_workspace(64, 8, 128) >= 128 * 4 + 129 * 4
    assert lib.moe355_gmm1_swiglu_quant_workspace(512, 1536, 2048, 128) >= 512 * 768 * 4


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from vllm_ascend_amd import _lib

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libmoe355.so"))
    with pytest.raises(ImportError, match="no CPU or PyTorch fallback"):
        _lib.load()


def test_package_never_touches_the_checker():
    pkg = os.path.join(ROOT, "vllm_ascend_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower(), f"{f} mentions the checker"


def test_custom_ops_schemas_and_meta():
    from vllm_ascend_amd.custom_ops import enable_custom_op

    assert enable_custom_op()
    ops = torch.ops._C_ascend
    x = torch.empty(5, 128, device="meta")
    y, idx, out = ops.moe_gating_top_k(x, k=8, k_group=1, group_count=1, group_select_mode=1, renorm=1, norm_type=0,
                                       out_flag=False, routed_scaling_factor=1.0, eps=1e-20, bias_opt=None)
    assert y.shape == (5, 8) and idx.dtype == torch.int32 and out.shape == (5, 128) and out.dtype == torch.float32
    xi = torch.empty(16, 64, dtype=torch.int8, device="meta")
    w = torch.empty(4, 64, 128, dtype=torch.int8, device="meta")
    o, s, off = ops.grouped_matmul_swiglu_quant_weight_nz(
        x=xi, weight=w, weight_scale=torch.empty(4, 128, device="meta"), x_scale=torch.empty(16, device="meta"),
        group_list=torch.empty(4, dtype=torch.int64, device="meta"))
    assert o.shape == (16, 64) and o.dtype == torch.int8 and s.shape == (16,) and s.dtype == torch.float32
    o, s = ops.npu_dequant_swiglu_quant(torch.empty(3, 256, dtype=torch.int32, device="meta"), quant_mode=1)
    assert o.shape == (3, 128) and s.shape == (3,)
    # CPU tensors are refused: only the HIP kernels exist
    with pytest.raises(NotImplementedError):
        ops.moe_gating_top_k(torch.zeros(5, 128), k=8, k_group=1, group_count=1, group_select_mode=1, renorm=1,
                             norm_type=0, out_flag=False, routed_scaling_factor=1.0, eps=1e-20)


def test_gating_argument_checks_match_the_reference_adapter():
    """Messages of csrc/moe/moe_gating_top_k/moe_gating_top_k_torch_adpt.h:33-48."""
    from vllm_ascend_amd.custom_ops import _check_gating

    with pytest.raises(RuntimeError, match="The x should be 2D"):
        _check_gating(torch.zeros(8), None)
    with pytest.raises(RuntimeError, match="tensor expected but got a tensor with dtype"):
        _check_gating(torch.zeros(2, 8, dtype=torch.int32), None)
    with pytest.raises(RuntimeError, match="The dtype of x and bias should be same"):
        _check_gating(torch.zeros(2, 8), torch.zeros(8, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError, match="The bias should be 1D"):
        _check_gating(torch.zeros(2, 8), torch.zeros(1, 8))
    with pytest.raises(RuntimeError, match="The bias first dim should be same as x second dim"):
        _check_gating(torch.zeros(2, 8), torch.zeros(4))


def test_cumsum_group_list_known_answers():
    """Vectors of tests/ut/ops/test_moe_mlp.py:31-62."""
    from vllm_ascend_amd.fused_moe.moe_mlp import cumsum_group_list

    k = KATS["cumsum_group_list"]
    lists = {0: torch.tensor(k["type0_cumsum"]), 1: torch.tensor(k["type1_count"]),
             2: torch.tensor([[1, 2], [2, 1], [0, 0], [0, 0]])}
    for src, dst in k["supported"]:
        assert torch.equal(cumsum_group_list(lists[src], src, dst, expert_num=4), lists[dst])
    with pytest.raises(ValueError, match=r"group_list_type should be in \[0, 1, 2\], but received"):
        cumsum_group_list(lists[0], 4, 0)
    for src, dst in k["unsupported"]:
        with pytest.raises(NotImplementedError, match="This feature is under development."):
            cumsum_group_list(lists[0], src, dst)
    # sparse pairs -> running sum
    sparse = torch.tensor([[1, 2], [3, 1]])
    assert cumsum_group_list(sparse, 2, 0, active_num=3, expert_num=4).tolist() == [0, 2, 2, 3]


def test_scheme_weight_specs_match_the_reference():
    """Names and shapes of vllm_ascend/quantization/methods/w8a8_dynamic.py:198-222."""
    from vllm_ascend_amd.quant_type import QuantType
    from vllm_ascend_amd.quantization import get_scheme_class

    scheme = get_scheme_class("W8A8_DYNAMIC", "moe")()
    assert scheme.quant_type == QuantType.W8A8 and scheme.supports_eplb
    w = scheme.get_weight(8, 1408, 1024, torch.bfloat16)
    assert w["w13_weight"].shape == (8, 2816, 1024) and w["w13_weight"].dtype == torch.int8
    assert w["w2_weight"].shape == (8, 1024, 1408) and w["w2_weight"].dtype == torch.int8
    q = scheme.get_dynamic_quant_param(8, 1408, 1024, torch.bfloat16)
    assert q["w13_weight_scale"].shape == (8, 2816, 1) and q["w13_weight_scale"].dtype == torch.bfloat16
    assert q["w2_weight_scale"].shape == (8, 1024, 1) and q["w13_weight_offset"].shape == (8, 2816, 1)
    with pytest.raises(NotImplementedError):
        get_scheme_class("W8A8_MXFP8", "moe")


def test_unsupported_options_raise_by_name():
    from vllm_ascend_amd.fused_moe.contracts import FusedMoEConfig, build_fused_experts_input, build_token_dispatch_input
    from vllm_ascend_amd.fused_moe.token_dispatcher import TokenDispatcherWithAllGather
    from vllm_ascend_amd.quant_type import QuantType

    with pytest.raises(NotImplementedError, match="one GPU"):
        FusedMoEConfig(num_experts=8, experts_per_token=2, hidden_dim=64, intermediate_size_per_partition=64,
                       ep_size=2)
    disp = TokenDispatcherWithAllGather(top_k=2, num_experts=8, num_local_experts=8)
    base = dict(hidden_states=torch.zeros(4, 64, dtype=torch.bfloat16), topk_weights=torch.zeros(4, 2),
                topk_ids=torch.zeros(4, 2, dtype=torch.int32), w1=[None], w2=[None], quant_type=QuantType.W8A8)
    for kw, pat in ((dict(expert_map=torch.arange(8)), "expert_map"), (dict(mc2_mask=torch.ones(4)), "mc2_mask")):
        inp = build_token_dispatch_input(fused_experts_input=build_fused_experts_input(**base, **kw))
        with pytest.raises(NotImplementedError, match=pat):
            disp.token_dispatch(inp)
    # pertoken_scale is honoured, for the int8 hidden states it belongs to (moe_mlp.py:226-242)
    inp = build_token_dispatch_input(fused_experts_input=build_fused_experts_input(
        **base, pertoken_scale=torch.ones(4)))
    with pytest.raises(ValueError, match="int8 hidden states"):
        disp.token_dispatch(inp)
    from vllm_ascend_amd.fused_moe.moe_mlp import quant_apply_mlp

    with pytest.raises(NotImplementedError, match="relu2"):
        quant_apply_mlp(torch.zeros(1, 8), None, None, None, None, torch.zeros(1), activation="relu2")
    with pytest.raises(NotImplementedError, match="swigluoai"):
        quant_apply_mlp(torch.zeros(1, 8), None, None, None, None, torch.zeros(1), activation="gelu", swiglu_alpha=1.7)


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys

    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "ONE GPU" in r.stderr


def test_w4a8_scheme_specs_and_argument_checks():
    """Parameter names of vllm_ascend/quantization/methods/w4a8.py:146-196 (one int4 value per int8) with the
    group dimension of the scales last; group sizes the kernels cannot take are refused at construction."""
    from vllm_ascend_amd.quant_type import QuantType
    from vllm_ascend_amd.quantization import get_scheme_class

    cls = get_scheme_class("W4A8_DYNAMIC", "moe")
    scheme = cls(group_size=256)
    assert scheme.quant_type == QuantType.W4A8
    w = scheme.get_weight(4, 512, 1024, torch.bfloat16)
    assert w["w13_weight"].shape == (4, 1024, 1024) and w["w13_weight"].dtype == torch.int8
    assert w["w2_weight"].shape == (4, 1024, 512)
    q = scheme.get_dynamic_quant_param(4, 512, 1024, torch.bfloat16)
    assert q["w13_weight_scale"].shape == (4, 1024, 4) and q["w2_weight_scale"].shape == (4, 1024, 2)
    q0 = cls(group_size=0).get_dynamic_quant_param(4, 512, 1024, torch.bfloat16)
    assert q0["w13_weight_scale"].shape == (4, 1024, 1) and q0["w2_weight_scale"].shape == (4, 1024, 1)
    for bad in (-64, 32, 100):
        with pytest.raises(ValueError, match="group_size"):
            cls(group_size=bad)


def test_dense_quant_matmul_argument_checks():
    """npu_quant_matmul stands in for the call in vllm_ascend/ops/fused_moe/shared_experts.py:262-301: what it
    cannot do is refused by name before any kernel is launched."""
    from vllm_ascend_amd import npu_ops

    x = torch.zeros(2, 64, dtype=torch.int8)
    w = torch.zeros(64, 128, dtype=torch.int8)
    s = torch.ones(128)
    with pytest.raises(NotImplementedError, match="offset / bias"):
        npu_ops.npu_quant_matmul(x, w, s, bias=torch.zeros(128))
    with pytest.raises(NotImplementedError, match="int8"):
        npu_ops.npu_quant_matmul(x.to(torch.bfloat16), w, s)
    with pytest.raises(NotImplementedError, match="pertoken_scale"):
        npu_ops.npu_quant_matmul(x, w, s, output_dtype=torch.bfloat16)
    with pytest.raises(NotImplementedError, match="output_dtype"):
        npu_ops.npu_quant_matmul(x, w, s, pertoken_scale=torch.ones(2), output_dtype=torch.float32)
    with pytest.raises(RuntimeError):   # CPU tensors never reach a kernel: there is no host fallback
        npu_ops.npu_quant_matmul(x, w, s, output_dtype=torch.int32)


def test_grouped_gemm_launchers_check_their_operands_on_the_host():
    """The C ABI takes raw pointers: a scale in the model dtype, a short group list or a mis-shaped x must raise
    in Python instead of being read out of bounds on the device.  (The checks run before the device test, so
    CPU tensors reach them.)"""
    from vllm_ascend_amd import kernels as K

    E, n, k, rows = 4, 128, 64, 8
    x = torch.zeros(rows, k, dtype=torch.int8)
    w = torch.zeros(E, k, n, dtype=torch.int8)
    s = torch.ones(E, n)
    xs = torch.ones(rows)
    gl = torch.tensor([2, 2, 2, 2])
    good = dict(x=x, weight_nz=w, weight_scale=s, x_scale=xs, group_list=gl)

    def gmm1(**kw):
        a = {**good, **kw}
        return K.gmm1_swiglu_quant(a["x"], a["weight_nz"], a["weight_scale"], a["x_scale"], a["group_list"], 1, n, k)

    with pytest.raises(TypeError, match="x must be int8"):
        gmm1(x=x.to(torch.bfloat16))
    with pytest.raises(ValueError, match=r"x must be \[rows, K"):
        gmm1(x=torch.zeros(rows, k + 32, dtype=torch.int8))
    with pytest.raises(ValueError, match="one entry per expert"):
        gmm1(group_list=gl[:3])
    with pytest.raises(TypeError, match="x_scale must be float32"):
        gmm1(x_scale=xs.to(torch.bfloat16))
    with pytest.raises(ValueError, match="one scale per row"):
        gmm1(x_scale=torch.ones(rows - 1))
    with pytest.raises(TypeError, match="weight scale must be float32"):
        gmm1(weight_scale=s.to(torch.bfloat16))
    with pytest.raises(ValueError, match="weight scale holds"):
        gmm1(weight_scale=torch.ones(E, n // 2))
    with pytest.raises(ValueError, match="weight holds"):
        gmm1(weight_nz=torch.zeros(E, k, n // 2, dtype=torch.int8))
    with pytest.raises(RuntimeError, match="no CPU implementation"):  # everything else right: refused as a CPU tensor
        gmm1()
    w2 = torch.zeros(E, n // 2, 64, dtype=torch.int8)
    q1 = torch.zeros(rows, n // 2, dtype=torch.int8)
    with pytest.raises(TypeError, match="per_token_scale must be float32"):
        K.gmm2_dequant(q1, w2, torch.ones(E, 64), xs.double(), gl, 1, 64, n // 2)
    with pytest.raises(ValueError, match="one entry per expert"):
        K.gmm2_dequant(q1, w2, torch.ones(E, 64), xs, gl[:2], 1, 64, n // 2)
    with pytest.raises(TypeError, match="weight scale must be float32"):
        K.gmm2_dequant(q1, w2, torch.ones(E, 64, dtype=torch.bfloat16), xs, gl, 1, 64, n // 2)
    w4 = torch.zeros(E, n * k // 2, dtype=torch.uint8)
    with pytest.raises(ValueError, match="weight scale holds"):
        K.gmm1_swiglu_quant_w4(x, w4, torch.ones(E, 1, n), 32, xs, gl, 1, n, k)  # group 32: two groups expected


def test_expert_tensor_lists_keep_their_address_tables():
    """One table per list, built when the list is created and kept for its lifetime (a captured HIP graph holds the
    table's address): many layers, and many lookups, never rebuild or evict a table; replacing an expert rewrites
    one entry of the same table."""
    from vllm_ascend_amd.kernels import ExpertTensorList, _as_expert_list

    layers = []
    for layer in range(40):  # more per-expert-list layers than Qwen3-30B-A3B or DeepSeek-V3 ever evicted before
        lists = [ExpertTensorList([torch.zeros(8, 16, dtype=torch.int8) for _ in range(6)], "w") for _ in range(4)]
        layers.append((lists, [lst.table for lst in lists]))
    for _ in range(3):
        for lists, tables in layers:
            for lst, tab in zip(lists, tables):
                assert _as_expert_list(lst, "w", torch.int8) is lst and lst.table is tab
                assert tab.tolist() == [t.data_ptr() for t in lst]
    lst, tab = layers[0][0][0], layers[0][1][0]
    new = torch.ones(8, 16, dtype=torch.int8)
    lst[2] = new
    assert lst.table is tab and tab[2].item() == new.data_ptr() and lst[2] is new
    with pytest.raises(RuntimeError, match=r"one\s+shape"):
        lst[1] = torch.ones(8, 8, dtype=torch.int8)
    with pytest.raises(TypeError, match="fixed"):
        lst.append(new)
    # a plain list gets a table of its own, for the one call
    plain = [torch.zeros(8, 16, dtype=torch.int8) for _ in range(3)]
    assert isinstance(_as_expert_list(plain, "w", torch.int8), ExpertTensorList)
    with pytest.raises(RuntimeError, match="must be torch.float32"):
        _as_expert_list(lst, "w", torch.float32)


def test_force_load_balance_replaces_the_ids_only():
    """Profile-run routing (vllm_ascend/ops/fused_moe/routed_experts.py:484-492): k distinct random experts per
    token; exercised here on the replacement step itself (the gating kernel needs the GPU)."""
    from vllm_ascend_amd.fused_moe.router import AscendFusedTopKRouter

    r = AscendFusedTopKRouter(4, 32)
    w = torch.rand(10, 4).to(torch.bfloat16)
    ids = torch.zeros(10, 4, dtype=torch.int32)
    r._compute_routing = lambda *a, **k: (w, ids)
    torch.manual_seed(0)
    w2, ids2 = r.select_experts(torch.zeros(10, 8, dtype=torch.bfloat16), torch.zeros(10, 32),
                                enable_force_load_balance=True)
    assert torch.equal(w2, w) and ids2.dtype == ids.dtype and ids2.shape == ids.shape
    assert int(ids2.min()) >= 0 and int(ids2.max()) < 32
    assert all(len(set(row.tolist())) == 4 for row in ids2)          # distinct experts per token
    assert len(set(ids2.reshape(-1).tolist())) > 8                    # spread over the experts
    w3, ids3 = r.select_experts(torch.zeros(10, 8, dtype=torch.bfloat16), torch.zeros(10, 32))
    assert ids3 is ids


def test_expert_load_from_both_group_list_forms():
    """Counts (type 1) and running totals (type 0) must add the same loads (routed_experts.py:571-587)."""
    import types

    import torch

    from vllm_ascend_amd.fused_moe.contracts import FusedExpertsResult
    from vllm_ascend_amd.fused_moe.layer import AscendRoutedExperts

    counts = torch.tensor([3, 0, 5, 1], dtype=torch.int64)
    for multi_stage in (False, True):
        holder = types.SimpleNamespace(
            multi_stage=multi_stage, num_iter=3, load_counter=torch.zeros((), dtype=torch.int32),
            moe_load=torch.zeros((3, 4), dtype=torch.int32) if multi_stage else torch.zeros(4, dtype=torch.int64))
        for glt, tokens in ((1, counts), (0, counts.cumsum(0)), (1, counts), (0, counts.cumsum(0))):
            res = FusedExpertsResult(routed_out=torch.zeros(1), group_list_type=glt, expert_tokens=tokens)
            AscendRoutedExperts._record_expert_load(holder, res)
        if multi_stage:
            assert holder.moe_load.tolist() == [(2 * counts).tolist(), counts.tolist(), counts.tolist()]
            assert int(holder.load_counter) == 4
        else:
            assert holder.moe_load.tolist() == (4 * counts).tolist()
    res = FusedExpertsResult(routed_out=torch.zeros(1))
    try:
        AscendRoutedExperts._record_expert_load(holder, res)
    except AssertionError as e:
        assert "should not be None when dynamic_eplb is enabled" in str(e)
    else:
        raise AssertionError("a result without expert_tokens must be refused")

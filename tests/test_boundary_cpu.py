"""CPU-side checks of the drop-in boundary: the C-ABI library loads and exports
every symbol include/ts_hip.h declares, the torch operators are registered
under the reference's names with the reference's schemas, and host-side error
behaviour. No GPU compute is launched here."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "ts_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ts_[a-z_0-9]+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    syms = _declared_symbols()
    for name in ("ts_scatter", "ts_segment_csr", "ts_segment_coo", "ts_gather_csr", "ts_gather_coo",
                 "ts_segment_mean_csr_backward", "ts_segment_mean_coo_backward", "ts_arg_backward",
                 "ts_hip_version", "ts_error_string"):
        assert name in syms


def test_library_exports_every_declared_symbol():
    from pytorch_scatter_amd import capi
    lib = capi.lib()
    for name in _declared_symbols():
        assert hasattr(lib, name), name
    assert sorted(capi.EXPORTS) == _declared_symbols()
    assert capi.hip_version() > 0
    assert capi.lib().ts_error_string(3).decode().startswith("workspace")


def test_status_codes_without_a_gpu():
    from pytorch_scatter_amd import capi
    lib = capi.lib()
    i = ctypes.c_int64
    # unknown dtype / negative size / unsupported reduce are rejected before any launch
    assert lib.ts_gather_csr(None, None, None, i(1), i(2), i(2), i(2), i(0), 99, None) == 1
    assert lib.ts_gather_csr(None, None, None, i(1), i(-2), i(2), i(2), i(0), 0, None) == 1
    assert lib.ts_segment_csr(None, None, None, None, i(1), i(2), i(2), i(2), i(0), 0, capi.MUL,
                              None, ctypes.c_size_t(0), None) == 2
    # null buffers with non-empty shapes
    assert lib.ts_gather_csr(None, None, None, i(1), i(2), i(2), i(2), i(0), 0, None) == 1
    # empty problems succeed without touching anything
    assert lib.ts_gather_csr(None, None, None, i(1), i(0), i(0), i(4), i(0), 0, None) == 0
    assert lib.ts_scatter(None, None, None, None, i(1), i(0), i(4), i(0), i(0), i(1), i(0), 0, capi.SUM, 0, None) == 0
    # workspace sizes are reported for valid shapes and grow with the number of tiles
    f = lib.ts_segment_csr_workspace_bytes
    small = f(i(1), i(1000), i(5000), i(64), 0, capi.SUM)
    big = f(i(1), i(100000), i(5000000), i(64), 0, capi.SUM)
    assert 0 < small < big
    assert f(i(1), i(1000), i(5000), i(64), 0, capi.MAX) > small


REF_SCHEMAS = {
    # inferred from the C++ signatures registered in csrc/scatter.cpp:272-277,
    # segment_coo.cpp:240-246, segment_csr.cpp:233-239, version.cpp:41-42
    "cuda_version": "() -> int",
    "scatter_sum": "(Tensor _0, Tensor _1, int _2, Tensor? _3, int? _4) -> Tensor",
    "scatter_mul": "(Tensor _0, Tensor _1, int _2, Tensor? _3, int? _4) -> Tensor",
    "scatter_mean": "(Tensor _0, Tensor _1, int _2, Tensor? _3, int? _4) -> Tensor",
    "scatter_min": "(Tensor _0, Tensor _1, int _2, Tensor? _3, int? _4) -> (Tensor, Tensor)",
    "scatter_max": "(Tensor _0, Tensor _1, int _2, Tensor? _3, int? _4) -> (Tensor, Tensor)",
    "segment_sum_coo": "(Tensor _0, Tensor _1, Tensor? _2, int? _3) -> Tensor",
    "segment_mean_coo": "(Tensor _0, Tensor _1, Tensor? _2, int? _3) -> Tensor",
    "segment_min_coo": "(Tensor _0, Tensor _1, Tensor? _2, int? _3) -> (Tensor, Tensor)",
    "segment_max_coo": "(Tensor _0, Tensor _1, Tensor? _2, int? _3) -> (Tensor, Tensor)",
    "gather_coo": "(Tensor _0, Tensor _1, Tensor? _2) -> Tensor",
    "segment_sum_csr": "(Tensor _0, Tensor _1, Tensor? _2) -> Tensor",
    "segment_mean_csr": "(Tensor _0, Tensor _1, Tensor? _2) -> Tensor",
    "segment_min_csr": "(Tensor _0, Tensor _1, Tensor? _2) -> (Tensor, Tensor)",
    "segment_max_csr": "(Tensor _0, Tensor _1, Tensor? _2) -> (Tensor, Tensor)",
    "gather_csr": "(Tensor _0, Tensor _1, Tensor? _2) -> Tensor",
}


def _normalise(schema: str) -> str:
    s = str(schema).split("(", 1)[1]
    s = "(" + s
    return re.sub(r"(Tensor|int) _\d+(?=[,)]\s*$|\)$|, Tensor _\d+\)$)", r"\1", re.sub(r"-> \(?(.*?)\)?$", lambda m: "-> " + (
        "(" + ", ".join(t.split(" ")[0] for t in m.group(1).split(", ")) + ")" if "," in m.group(1) else m.group(1).split(" ")[0]), s))


@pytest.mark.parametrize("name", sorted(REF_SCHEMAS))
def test_operator_is_registered_with_reference_schema(name):
    import pytorch_scatter_amd  # noqa: F401  (registers torch.ops.torch_scatter.*)
    op = getattr(torch.ops.torch_scatter, name)
    assert _normalise(op.default._schema) == REF_SCHEMAS[name]


def test_python_surface_matches_reference_names():
    import pytorch_scatter_amd as ts
    for name in ["scatter_sum", "scatter_add", "scatter_mul", "scatter_mean", "scatter_min", "scatter_max",
                 "scatter", "segment_sum_csr", "segment_add_csr", "segment_mean_csr", "segment_min_csr",
                 "segment_max_csr", "segment_csr", "gather_csr", "segment_sum_coo", "segment_add_coo",
                 "segment_mean_coo", "segment_min_coo", "segment_max_coo", "segment_coo", "gather_coo",
                 "scatter_std", "scatter_logsumexp", "scatter_softmax", "scatter_log_softmax"]:
        assert callable(getattr(ts, name)), name
    assert ts.hip_version == torch.ops.torch_scatter.cuda_version()


def test_wrappers_are_scriptable():
    import pytorch_scatter_amd as ts
    for fn in (ts.scatter_sum, ts.scatter_max, ts.segment_mean_csr, ts.segment_min_coo, ts.gather_csr,
               ts.gather_coo, ts.scatter, ts.segment_csr, ts.segment_coo):
        torch.jit.script(fn)


def test_cpu_tensors_fail_loudly():
    import pytorch_scatter_amd as ts
    src = torch.ones(4)
    index = torch.tensor([0, 1, 0, 1])
    with pytest.raises(RuntimeError, match="must be CUDA tensor"):
        ts.scatter_sum(src, index)
    with pytest.raises(RuntimeError, match="must be CUDA tensor"):
        ts.segment_csr(src, torch.tensor([0, 2, 4]))
    with pytest.raises(RuntimeError, match="must be CUDA tensor"):
        ts.gather_coo(src, index.sort()[0])
    with pytest.raises(ValueError):
        ts.scatter(src, index, reduce="median")
    with pytest.raises(ValueError):
        ts.segment_csr(src, index, reduce="median")


def test_added_operators_and_index_reuse_without_a_gpu():
    """The operators this library adds are registered, their wrappers script, fail loudly on CPU tensors, and
    the index-reuse front-end never touches a call it is not meant for (CPU tensors, switched off)."""
    import pytorch_scatter_amd as ts
    from pytorch_scatter_amd import index_reuse
    for name in ("scatter_softmax", "scatter_logsumexp", "scatter_std", "index_to_indptr", "indptr_to_index",
                 "sort_index", "scatter_sorted"):
        assert hasattr(torch.ops.torch_scatter, name), name
    for fn in (ts.scatter_mean, ts.scatter_min, ts.scatter_add, ts.scatter_std, ts.scatter_softmax,
               ts.scatter_logsumexp, ts.index_to_indptr, ts.indptr_to_index):
        torch.jit.script(fn)
    index = torch.tensor([0, 1, 0, 1])
    with pytest.raises(RuntimeError, match="must be CUDA tensor"):
        ts.index_to_indptr(index.sort()[0], 2)
    with pytest.raises(RuntimeError, match="must be CUDA tensor"):
        ts.SortedIndex(index, 2)
    assert not ts.index_reuse_enabled()
    src = torch.ones(4, 32)
    assert index_reuse.plan_for(src, index, 0, None, 2) is None
    ts.enable_index_reuse(max_plans=2)
    try:
        assert index_reuse.plan_for(src, index, 0, None, 2) is None      # CPU tensors never qualify
        assert index_reuse.plan_for(src, index, 0, None, 2) is None
        assert len(index_reuse._cache) == 0
        with pytest.raises(RuntimeError, match="must be CUDA tensor"):   # and still fail loudly
            ts.scatter_sum(src, index, 0, None, 2)
    finally:
        ts.disable_index_reuse()
    assert not ts.index_reuse_enabled()


def test_product_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "pytorch_scatter_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".cpp", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "ts_oracle" not in text and "oracle/" not in text, f

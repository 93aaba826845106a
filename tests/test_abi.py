"""The C-ABI library loads without a GPU and exports every symbol include/*.h declares; the ctypes
signature table of the host package names exactly those symbols.  No compute calls here."""
import ctypes
import glob
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    names = set()
    for h in glob.glob(os.path.join(ROOT, "include", "*.h")):
        text = re.sub(r"/\*.*?\*/", "", open(h).read(), flags=re.S)
        names |= set(re.findall(r"\b(om_[a-z0-9_]+)\s*\(", text))
    return names


def test_header_declares_the_path():
    d = _declared()
    for must in ("om_adamw_step", "om_moe_sort", "om_route_softmax_topk", "om_route_sigmoid_group_topk",
                 "om_index_add", "om_index_gather", "om_compute_partial_token_counts",
                 "om_compute_input_and_output_indices", "om_shuffle_sub_matrix_reduce",
                 "om_reduce_ggemm_output", "om_reduce_ggemm_output_backward", "om_grouped_gemm_fwd",
                 "om_grouped_gemm_dgrad", "om_grouped_gemm_wgrad", "om_merged_mlp_gate_up_fwd"):
        assert must in d


def test_library_exports_every_declared_symbol():
    from optimus import _native
    assert os.path.exists(_native.LIB_PATH), "build the library first: python optimus-lm_amd/build.py"
    handle = ctypes.CDLL(_native.LIB_PATH)
    for name in sorted(_declared()):
        assert hasattr(handle, name), f"{name} declared in include/ but not exported"


def test_ctypes_table_matches_header():
    from optimus import _native
    assert set(_native.SIGNATURES) == _declared()


def test_identity_calls_without_gpu():
    from optimus import _native
    lib = _native.lib()
    assert lib.om_version() >= 100
    assert lib.om_arch() == b"gfx950"
    assert b"NULL" in lib.om_strerror(-1)
    assert lib.om_moe_sort_workspace_bytes(16384, 8, 64) > 0


def test_no_cpu_fallback():
    """Host wrappers refuse CPU tensors instead of computing elsewhere."""
    import torch
    import pcl_xpu_customops as ops
    from optimus import _native
    x = torch.zeros(4, 8)
    with pytest.raises(_native.NativeLibraryError):
        ops.index_gather(x, torch.zeros(4, dtype=torch.int32), torch.empty(4, 8))
    from optimus.optimizers import adamw_step_
    z = torch.zeros(8)
    with pytest.raises(_native.NativeLibraryError):
        adamw_step_(z.bfloat16(), z.bfloat16(), z, z.clone(), z.clone(), 1, 1e-3, 0.9, 0.95, 1e-8, 0.1)


def test_product_never_imports_oracle():
    """Nothing under the product package may import, load or execute the oracle."""
    pkg = os.path.join(ROOT, "optimus-lm_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f), errors="ignore").read()
                assert "oracle" not in text.lower().replace("oracle's", ""), os.path.join(dirpath, f)

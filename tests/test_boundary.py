"""The C-ABI library loads and exports every symbol the header declares; host-side argument
checking of the C ABI and of the Python operators (no GPU needed: nothing is launched)."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "pypto_amd", "libpypto_amd_sfa.so")
HEADER = os.path.join(ROOT, "include", "pypto_amd_sfa.h")


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(LIB):
        from pypto_amd.build import build_all
        build_all()
    return ctypes.CDLL(LIB)


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pto_\w+)\s*\(", text)))


def test_header_symbols_are_exported(lib):
    names = _declared()
    assert {"pto_sfa_quant_launch", "pto_sfa_quant_workspace_bytes", "pto_li_decode_launch",
            "pto_li_decode_workspace_bytes", "pto_li_prolog_quant_launch", "pto_li_prolog_quant_workspace_bytes",
            "pto_mla_prolog_quant_launch", "pto_mla_prolog_quant_workspace_bytes",
            "pto_last_error", "pto_version"} <= set(names)
    for n in names:
        assert hasattr(lib, n), n


def test_version_and_error_string(lib):
    lib.pto_version.restype = ctypes.c_char_p
    lib.pto_last_error.restype = ctypes.c_char_p
    assert re.fullmatch(rb"\d+\.\d+\.\d+", lib.pto_version())
    # the revision of the argument structs the library was built with is the one the header states
    declared = int(re.search(r"#define\s+PTO_ABI_REVISION\s+(\d+)", open(HEADER).read()).group(1))
    assert lib.pto_abi_revision() == declared
    n = ctypes.c_size_t(0)
    assert lib.pto_sfa_quant_workspace_bytes(None, ctypes.byref(n)) == -1
    assert b"NULL" in lib.pto_last_error()


def test_pybind_workspace_and_argument_errors():
    from pypto_amd import _native
    C = _native.load()
    # 32 rows x 8 splits x 128 heads x (512 fp16 + 2 fp32)
    assert C.sfa_quant_workspace_bytes(32, 1, 128, 1, 2048, 128, 512, 1 << 20, 0.04, 8) == 32 * 8 * 128 * (512 * 2 + 8)
    # more rows than compute units, a cache much larger than the selections: neither split nor de-quantised copy
    assert C.sfa_quant_workspace_bytes(4096, 1, 128, 1, 2048, 128, 32, 1 << 21, 0.04, 0) == 0
    # the automatic split (a host without a device plans for 256 compute units in 8 XCDs): 32 rows in 8 pieces each;
    # 200 rows whole; 300 rows as 256 whole rows and the other 44 in 5 pieces each; 260 rows as 256 whole rows and
    # the other 4 in 16 pieces (a piece keeps at least four tiles of 32 keys)
    assert C.sfa_quant_workspace_bytes(32, 1, 128, 1, 2048, 128, 512, 1 << 21, 0.04, 0) == 32 * 8 * 128 * (512 * 2 + 8)
    assert C.sfa_quant_workspace_bytes(200, 1, 128, 1, 2048, 128, 32, 1 << 21, 0.04, 0) == 0
    assert C.sfa_quant_workspace_bytes(300, 1, 128, 1, 2048, 128, 32, 1 << 21, 0.04, 0) == 44 * 5 * 128 * (512 * 2 + 8)
    assert C.sfa_quant_workspace_bytes(260, 1, 128, 1, 2048, 128, 32, 1 << 21, 0.04, 0) == 4 * 16 * 128 * (512 * 2 + 8)
    # prefill-shaped (every cache row selected by many query rows): one bf16 copy of the 4096 cache rows
    assert C.sfa_quant_workspace_bytes(4096, 1, 128, 1, 2048, 128, 32, 4096, 0.04, 0) == 4096 * 512 * 2
    assert C.li_decode_workspace_bytes(4, 4, 64, 128, 1024, 128, 256, 2048, 0, 0, 0) == 4 * (32768 + 2048) * 4
    # prolog: 4 int32 partial projections [t, 8192] + 112 block sums [t, 192] fp32
    assert C.li_prolog_quant_workspace_bytes(8, 7168, 1536, 64, 1 << 20) == 4 * 8 * 8192 * 4 + 112 * 8 * 192 * 4
    with pytest.raises(ValueError):
        C.li_prolog_quant_workspace_bytes(8, 7168, 1280, 64, 1 << 20)                # q_lora_rank not supported
    with pytest.raises(ValueError):
        C.li_prolog_quant_workspace_bytes(8, 7100, 1536, 64, 1 << 20)                # h not a multiple of 64
    with pytest.raises(ValueError):
        C.li_prolog_quant_workspace_bytes(8, 7168, 1536, 65, 1 << 20)                # more than 64 heads
    # MLA prolog: 14 group sums [t, 1536 + 576] fp32 + 4 int32 partial projections [t, 128 * 192]
    assert C.mla_prolog_quant_workspace_bytes(8, 7168, 1536, 128, 1 << 16) == 14 * 8 * 2112 * 4 + 4 * 8 * 24576 * 4
    # from 9 tokens on the partial sums over the hidden axis may be the matrix-core form's ranges (up to fourteen, one
    # per block of 64 hidden rows at most): a 192-wide hidden axis is one group but three ranges
    assert C.mla_prolog_quant_workspace_bytes(150, 192, 512, 2, 1 << 16) == 3 * 150 * 1088 * 4 + 4 * 150 * 384 * 4
    assert C.mla_prolog_quant_workspace_bytes(32, 192, 512, 2, 1 << 16) == 3 * 32 * 1088 * 4 + 4 * 32 * 384 * 4
    assert C.mla_prolog_quant_workspace_bytes(15, 192, 512, 2, 1 << 16) == 3 * 15 * 1088 * 4 + 4 * 15 * 384 * 4
    assert C.mla_prolog_quant_workspace_bytes(8, 192, 512, 2, 1 << 16) == 1 * 8 * 1088 * 4 + 4 * 8 * 384 * 4
    with pytest.raises(ValueError, match="sum_mode"):                                # indexer prolog: sum_mode is 0, 1 or 2
        C.li_prolog_quant_launch(*([0] * 19), 0, 0, 8, 7168, 1536, 64, 1 << 20, 1e-6, 3, 0)
    with pytest.raises(ValueError):
        C.mla_prolog_quant_workspace_bytes(8, 7168, 1536, 127, 1 << 16)              # odd head count
    with pytest.raises(ValueError):
        C.mla_prolog_quant_workspace_bytes(8, 32768, 1536, 128, 1 << 16)             # hidden size beyond the limit
    with pytest.raises(ValueError):
        C.sfa_quant_workspace_bytes(1, 1, 128, 2, 2048, 128, 32, 4096, 0.04, 0)      # n_kv != 1
    with pytest.raises(ValueError):
        C.li_decode_workspace_bytes(4, 4, 32, 128, 1024, 128, 256, 2048, 0, 0, 0)    # 32 heads
    with pytest.raises(ValueError):
        C.li_decode_workspace_bytes(4, 4, 64, 128, 1024, 128, 256, 4096, 0, 0, 0)    # selected_count > 2048
    with pytest.raises(ValueError):
        C.li_decode_workspace_bytes(4, 4, 64, 128, 4096, 128, 2048, 2048, 0, 0, 0)   # longer than 128K
    with pytest.raises(ValueError):                                                  # NULL tensors
        C.sfa_quant_launch(0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 1, 1, 16, 1, 256, 128, 32, 4096, 0.04, 0, 0)


def test_from_torch_contract():
    import pypto_amd
    t = torch.zeros(4, 6)
    h = pypto_amd.from_torch(t, name="x", dynamic_axis=[0])
    assert h.shape == [4, 6] and h.dtype == torch.float32 and h.data_ptr == t.data_ptr() and h.name == "x"
    with pytest.raises(TypeError):
        pypto_amd.from_torch([1, 2, 3])
    with pytest.raises(RuntimeError):
        pypto_amd.from_torch(t.t())


def test_operators_refuse_cpu_tensors_loudly():
    """There is no CPU fallback behind the operator names."""
    import pypto_amd
    from pypto_amd.synthetic import gen_sfa_inputs, gen_indexer_inputs
    inp = gen_sfa_inputs(1, 1, 16, [256], topk=64, seed=0)
    out = torch.zeros(1, 1, 16, 512, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError):
        pypto_amd.sparse_flash_attention_quant_d(*inp.operator_tensors(), out, 16, 1, inp.softmax_scale, 64, 128,
                                                 inp.max_blocknum_perbatch, None)
    li = gen_indexer_inputs(1, 1, [256], selected_count=64, seed=0)
    with pytest.raises(RuntimeError):
        pypto_amd.lightning_indexer_decode(*li.operator_tensors(), None, None, 64)


def test_prolog_operators_refuse_cpu_tensors_and_unbuilt_variants():
    import pypto_amd
    from pypto_amd.synthetic import gen_indexer_prolog_inputs, gen_mla_prolog_inputs
    kw = dict(h=128, q_lora_rank=512, n_heads=2)
    lip = gen_indexer_prolog_inputs(1, 1, [130], seed=0, **kw)
    outs = (torch.zeros(1, 2, 128, dtype=torch.int8), torch.zeros(1, 2, 1, dtype=torch.float16), lip.k_cache,
            lip.k_cache_scale, torch.zeros(1, 2, dtype=torch.float16))
    with pytest.raises(RuntimeError):
        pypto_amd.lightning_indexer_prolog_quant(*lip.input_tensors(), *outs)
    with pytest.raises(ValueError):
        pypto_amd.lightning_indexer_prolog_quant(*lip.input_tensors(), *outs,
                                                 pypto_amd.IndexerPrologQuantAttr(layerout_key="BSND"))
    mla = gen_mla_prolog_inputs(1, 1, [130], seed=0, **kw)
    mouts = (torch.zeros(1, 512, dtype=torch.int8), torch.zeros(1, 1), torch.zeros(1, 2, 512, dtype=torch.bfloat16),
             torch.zeros(1, 2, 64, dtype=torch.bfloat16), mla.kv_cache, mla.kr_cache, mla.k_scale_cache)
    with pytest.raises(RuntimeError):
        pypto_amd.mla_prolog_quant_d(*mla.input_tensors(), *mouts, 1e-5, 1e-5, "PA_BSND", None, None)
    with pytest.raises(RuntimeError):                    # an accepted cache mode (the reference asserts "PA_BSND" or "PA_NZ"
        pypto_amd.mla_prolog_quant_d(*mla.input_tensors(), *mouts, 1e-5, 1e-5, "PA_NZ", None, None)   # and treats them alike)
    with pytest.raises(ValueError):
        pypto_amd.mla_prolog_quant_d(*mla.input_tensors(), *mouts, 1e-5, 1e-5, "BSND", None, None)
    args = list(mla.input_tensors())
    args[3] = None                                       # no dequant scale: the non-quantized up-projection
    with pytest.raises(ValueError):
        pypto_amd.mla_prolog_quant_d(*args, *mouts, 1e-5, 1e-5, "PA_BSND", None, None)


def test_cache_out_overlapping_cache_in_is_refused():
    """The prolog operators copy cache-in to cache-out unless they are the same tensor; two views that share
    memory without being the same range must not be copied onto each other."""
    import torch
    from pypto_amd.converter import copy_unless_same
    base = torch.arange(64, dtype=torch.int8)
    copy_unless_same(base[:32], base[:32], "k_int8")                 # same range: nothing happens
    other = torch.zeros(32, dtype=torch.int8)
    copy_unless_same(other, base[:32], "k_int8")                     # disjoint: copied
    assert torch.equal(other, base[:32])
    with pytest.raises(ValueError, match="overlap"):
        copy_unless_same(base[8:40], base[:32], "k_int8")

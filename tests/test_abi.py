"""The C-ABI library: loads, exports what the header declares, lays structs out
as the Python binding expects, and rejects bad calls before touching the GPU."""

import ctypes as C
import re
import shutil
import subprocess
from pathlib import Path

import pytest

from cppmega_mlx_amd import _lib

ROOT = Path(__file__).resolve().parents[1]
HEADER = ROOT / "include" / "cppmega_mi355.h"


def _declared_functions() -> list[str]:
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(cppmega_mi355_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    declared = _declared_functions()
    assert set(declared) == set(_lib.EXPORTED_SYMBOLS)
    for name in declared:
        assert hasattr(lib, name), name


def test_status_probe_reports_abi_and_arch():
    st = _lib.status()
    assert st["abi_version"] == _lib.ABI_VERSION == 1
    assert st["built_for"] == "gfx950"
    assert st["device_count"] >= 0


STRUCTS = {
    "cppmega_mi355_status_t": _lib.StatusStruct,
    "cppmega_mi355_topk_args_t": _lib.TopkArgs,
    "cppmega_mi355_indexer_args_t": _lib.IndexerArgs,
    "cppmega_mi355_head_gemm_args_t": _lib.HeadGemmArgs,
    "cppmega_mi355_dsa_loss_args_t": _lib.DsaLossArgs,
    "cppmega_mi355_sparse_mla_bwd_args_t": _lib.SparseMlaBwdArgs,
    "cppmega_mi355_dequant_block_args_t": _lib.DequantBlockArgs,
    "cppmega_mi355_sparse_mla_args_t": _lib.SparseMlaArgs,
    "cppmega_mi355_vecmat_args_t": _lib.VecmatArgs,
    "cppmega_mi355_quantize_args_t": _lib.QuantizeArgs,
    "cppmega_mi355_cache_append_args_t": _lib.CacheAppendArgs,
    "cppmega_mi355_causal_indices_args_t": _lib.CausalIndicesArgs,
    "cppmega_mi355_mask_indices_args_t": _lib.MaskIndicesArgs,
}


def _header_struct_fields() -> dict[str, list[str]]:
    """Field names, in order, of every ``typedef struct ... {...} name_t;`` in the header."""
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    found = {}
    for body, name in re.findall(r"typedef\s+struct\s+\w+\s*\{(.*?)\}\s*(\w+)\s*;", text, flags=re.S):
        names = []
        for decl in body.split(";"):
            decl = decl.strip()
            if not decl:
                continue
            for part in decl.split(","):
                names.append(re.search(r"(\w+)\s*(\[[^\]]*\])?\s*$", part.strip()).group(1))
        found[name] = names
    return found


def test_every_header_struct_has_a_ctypes_mirror_with_the_same_fields():
    header = _header_struct_fields()
    assert set(header) == set(STRUCTS)
    for ctype, struct in STRUCTS.items():
        assert [n for n, _ in struct._fields_] == header[ctype], ctype


@pytest.mark.skipif(shutil.which("gcc") is None, reason="gcc not available")
def test_struct_layouts_match_the_header(tmp_path):
    """Size of every struct and offset of every field, as a C compiler lays the header out."""
    lines = ['#include <stdio.h>', '#include <stddef.h>', f'#include "{HEADER}"', "int main(void){"]
    for ctype, struct in STRUCTS.items():
        lines.append(f'printf("{ctype} size %zu\\n", sizeof({ctype}));')
        for n, _ in struct._fields_:
            lines.append(f'printf("{ctype} {n} %zu\\n", offsetof({ctype}, {n}));')
    lines.append('printf("v1 size %zu\\n", (size_t)CPPMEGA_MI355_SPARSE_MLA_ARGS_V1_SIZE);')
    lines.append("return 0;}")
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout
    checked = 0
    for line in out.strip().splitlines():
        ctype, name, value = line.split()
        if ctype == "v1":
            assert _lib.SparseMlaArgs.sm_scale_dev.offset == int(value) == _lib.SPARSE_MLA_ARGS_V1_SIZE
            continue
        struct = STRUCTS[ctype]
        got = C.sizeof(struct) if name == "size" else getattr(struct, name).offset
        assert got == int(value), f"{ctype}.{name}: ctypes {got} != C {value}"
        checked += 1
    assert checked == sum(len(s._fields_) + 1 for s in STRUCTS.values())


def test_null_and_short_struct_are_rejected_with_the_bridge_codes():
    lib = _lib.load()
    assert lib.cppmega_mi355_status(None, 0) == _lib.ERR_NULL
    st = _lib.StatusStruct()
    assert lib.cppmega_mi355_status(C.byref(st), 4) == _lib.ERR_STRUCT_SIZE
    assert lib.cppmega_mi355_topk_select(None, 0, None) == _lib.ERR_NULL
    args = _lib.TopkArgs()
    args.struct_size = 8
    assert lib.cppmega_mi355_topk_select(C.byref(args), C.sizeof(args), None) == _lib.ERR_STRUCT_SIZE
    assert lib.cppmega_mi355_fp8_vecmat(None, 0, None) == _lib.ERR_NULL
    assert lib.cppmega_mi355_sparse_mla_fwd(None, 0, None) == _lib.ERR_NULL
    assert b"NULL" in lib.cppmega_mi355_error_string(_lib.ERR_NULL)


def test_first_abi_sparse_mla_struct_is_still_accepted():
    """A caller built before sm_scale_dev / has_sinks_dev / seq_kv_pitch were appended passes the
    shorter struct_size; anything shorter than that is rejected."""
    lib = _lib.load()
    a = _latent_mla_args()
    want = lib.cppmega_mi355_sparse_mla_select_kernel(C.byref(a), C.sizeof(a))
    assert want == _lib.MLA_KERNEL_MFMA
    a.seq_kv_pitch = 7                                   # below seq_kv: a shape error when it is read...
    assert lib.cppmega_mi355_sparse_mla_select_kernel(C.byref(a), C.sizeof(a)) == -_lib.ERR_SHAPE
    a.struct_size = _lib.SPARSE_MLA_ARGS_V1_SIZE         # ...and not read at all from a first-ABI caller
    assert lib.cppmega_mi355_sparse_mla_select_kernel(C.byref(a), _lib.SPARSE_MLA_ARGS_V1_SIZE) == want
    need = C.c_size_t(0)
    assert lib.cppmega_mi355_sparse_mla_workspace_bytes(C.byref(a), C.sizeof(a), C.byref(need)) == _lib.OK
    a.struct_size = _lib.SPARSE_MLA_ARGS_V1_SIZE - 8
    assert lib.cppmega_mi355_sparse_mla_workspace_bytes(C.byref(a), C.sizeof(a), C.byref(need)) == _lib.ERR_STRUCT_SIZE
    assert lib.cppmega_mi355_sparse_mla_select_kernel(C.byref(a), C.sizeof(a)) == -_lib.ERR_STRUCT_SIZE


def test_contract_violations_return_shape_and_dtype_codes_without_a_gpu():
    lib = _lib.load()
    fake = 0x1000  # never dereferenced: validation fails first
    t = _lib.TopkArgs()
    t.struct_size = C.sizeof(t)
    t.scores, t.indices, t.rows, t.width, t.row_stride, t.k = fake, fake, 2, 16, 16, 17
    assert lib.cppmega_mi355_topk_select(C.byref(t), C.sizeof(t), None) == _lib.ERR_SHAPE
    assert b"topk must be in [1, 16]" in lib.cppmega_mi355_last_error()
    t.k, t.score_dtype = 4, _lib.I32
    assert lib.cppmega_mi355_topk_select(C.byref(t), C.sizeof(t), None) == _lib.ERR_DTYPE
    t.score_dtype, t.width, t.row_stride, t.k = _lib.F32, 70000, 70000, 4
    assert lib.cppmega_mi355_topk_select(C.byref(t), C.sizeof(t), None) == _lib.ERR_UNSUPPORTED

    m = _lib.SparseMlaArgs()
    m.struct_size = C.sizeof(m)
    m.q = m.kv = m.indices = m.out = fake
    m.q_dtype = m.kv_dtype = m.out_dtype = _lib.BF16
    m.index_dtype = _lib.I32
    m.batch, m.seq_q, m.heads, m.kv_groups, m.seq_kv, m.topk, m.d_qk, m.d_v = 1, 1, 6, 4, 8, 4, 64, 64
    assert lib.cppmega_mi355_sparse_mla_fwd(C.byref(m), C.sizeof(m), None) == _lib.ERR_SHAPE
    assert b"not divisible by kv_group" in lib.cppmega_mi355_last_error()
    m.kv_groups, m.d_v = 2, 65
    assert lib.cppmega_mi355_sparse_mla_fwd(C.byref(m), C.sizeof(m), None) == _lib.ERR_SHAPE
    m.d_v, m.index_dtype = 64, _lib.F32
    assert lib.cppmega_mi355_sparse_mla_fwd(C.byref(m), C.sizeof(m), None) == _lib.ERR_DTYPE

    v = _lib.VecmatArgs()
    v.struct_size = C.sizeof(v)
    v.x = v.w = v.scale_w = v.out = fake
    v.m, v.n, v.k, v.x_dtype, v.out_dtype = 1, 8, 0, _lib.BF16, _lib.BF16
    assert lib.cppmega_mi355_fp8_vecmat(C.byref(v), C.sizeof(v), None) == _lib.ERR_SHAPE
    v.k, v.x_dtype = 16, _lib.E4M3
    assert lib.cppmega_mi355_fp8_vecmat(C.byref(v), C.sizeof(v), None) == _lib.ERR_NULL  # scale_x missing


def test_check_maps_codes_to_python_errors():
    with pytest.raises(ValueError):
        _lib.check(_lib.ERR_SHAPE, "op")
    with pytest.raises(TypeError):
        _lib.check(_lib.ERR_DTYPE, "op")
    with pytest.raises(_lib.NativeCallError) as info:
        _lib.check(_lib.ERR_LAUNCH, "op")
    assert info.value.code == _lib.ERR_LAUNCH
    _lib.check(_lib.OK, "op")


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", tmp_path / "nope.so")
    with pytest.raises(_lib.NativeLibraryError, match="no fallback"):
        _lib.load()


def _latent_mla_args(**over):
    """The decode layout (bf16 q, e4m3 latent + fp32/128 scales + bf16 rope), no buffers attached."""
    a = _lib.SparseMlaArgs()
    a.struct_size = C.sizeof(a)
    a.kernel = _lib.MLA_KERNEL_AUTO
    a.q_dtype, a.q_scale_kind = _lib.BF16, _lib.SCALE_NONE
    a.kv_dtype, a.kv_scale_kind, a.kv_scale_block = _lib.E4M3, _lib.SCALE_F32_BLOCK, 128
    a.rope_dtype, a.rope_dim = _lib.BF16, 64
    a.index_dtype, a.out_dtype = _lib.I32, _lib.BF16
    a.batch, a.seq_q, a.heads, a.kv_groups, a.seq_kv, a.topk = 32, 1, 128, 1, 65536, 2048
    a.d_qk, a.d_v, a.sm_scale = 576, 512, 576 ** -0.5
    for k, v in over.items():
        setattr(a, k, v)
    return a


def test_kernel_choice_and_workspace_for_the_latent_cache_layout():
    """Host-side plan of the shared-tile kernel (no GPU work): which kernel AUTO picks and what
    workspace the key splits need.  Key lists longer than 16 splits of 2048 keys are left to the
    scalar kernel (the combine step merges at most 16 splits)."""
    lib = _lib.load()
    need = C.c_size_t(0)
    a = _latent_mla_args()
    assert lib.cppmega_mi355_sparse_mla_select_kernel(C.byref(a), C.sizeof(a)) == _lib.MLA_KERNEL_MFMA
    assert lib.cppmega_mi355_sparse_mla_workspace_bytes(C.byref(a), C.sizeof(a), C.byref(need)) == 0
    # 32 queries x 2 head chunks x 4 key splits, each 64 heads x 512 channels bf16 + (max, sum) per head
    assert need.value == 32 * 2 * 4 * (64 * 512 * 2 + 64 * 2 * 4)
    a = _latent_mla_args(batch=1, seq_q=8192, seq_kv=8192)            # prefill: enough queries, no key splits
    assert lib.cppmega_mi355_sparse_mla_workspace_bytes(C.byref(a), C.sizeof(a), C.byref(need)) == 0 and need.value == 0
    # longer lists go to the 32-head tile kernel, whose split count stops at 16 and whose partials are
    # fp32 rows [B S, H, splits, 512 + 2]
    a = _latent_mla_args(batch=1, topk=40000, seq_kv=65536)
    assert lib.cppmega_mi355_sparse_mla_select_kernel(C.byref(a), C.sizeof(a)) == _lib.MLA_KERNEL_MFMA
    assert lib.cppmega_mi355_sparse_mla_workspace_bytes(C.byref(a), C.sizeof(a), C.byref(need)) == 0
    assert need.value == 128 * 16 * (512 + 2) * 4
    a = _latent_mla_args(batch=1, topk=32768)                            # exactly 16 splits of 2048 keys
    assert lib.cppmega_mi355_sparse_mla_select_kernel(C.byref(a), C.sizeof(a)) == _lib.MLA_KERNEL_MFMA
    assert lib.cppmega_mi355_sparse_mla_workspace_bytes(C.byref(a), C.sizeof(a), C.byref(need)) == 0
    assert need.value == 2 * 16 * (64 * 512 * 2 + 64 * 2 * 4)

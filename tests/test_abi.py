"""The C-ABI library loads and exports every entry point include/ohara_decode.h declares
(no compute call: this runs without a GPU)."""

import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "ohara_decode.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"^\s*(?:int|int64_t)\s+(ohara_[a-z0-9_]+)\s*\(", text, flags=re.M)
    assert len(names) >= 15
    return sorted(set(names))


def test_library_exports_every_declared_symbol():
    from ohara_amd import _lib

    assert os.path.exists(_lib.LIB_PATH), "build the library first: python -m ohara_amd.build"
    handle = ctypes.CDLL(_lib.LIB_PATH)
    missing = [n for n in declared_functions() if not hasattr(handle, n)]
    assert not missing, missing
    handle.ohara_abi_version.restype = ctypes.c_int
    assert handle.ohara_abi_version() >= 1


def test_python_prototypes_cover_the_header():
    from ohara_amd import _lib

    declared = set(declared_functions())
    bound = set(_lib._PROTOS)
    assert declared <= bound, declared - bound
    assert bound <= declared, bound - declared
    _lib.lib()  # binds argtypes; raises if a symbol is absent


def test_struct_layouts_match_the_header():
    """Field order/size of the ctypes mirrors of OharaLayer / OharaModel / OharaDecodeState."""
    from ohara_amd import _lib

    assert ctypes.sizeof(_lib.OharaLayer) == 6 * 8
    assert ctypes.sizeof(_lib.OharaModel) == 8 * 4 + 4 + 4 + 6 * 8
    assert _lib.OharaModel.token_emb.offset == 40
    assert ctypes.sizeof(_lib.OharaDecodeState) == 6 * 4 + 12 * 8 + 8 + 5 * 8 + 3 * 8
    assert _lib.OharaDecodeState.seq_pos.offset == 24 + 12 * 8 + 8 + 5 * 8
    assert _lib.OharaDecodeState.kv_int8.offset == 24 + 12 * 8 and _lib.OharaDecodeState.kvstats.offset == 24 + 13 * 8
    assert _lib.OharaDecodeState.xn.offset == 24 + 5 * 8
    assert _lib.OharaDecodeState.ids.offset == 24
    assert ctypes.sizeof(_lib.OharaBitLayer) == 7 * 8 + 7 * 8 + 8 * 4 + 2 * 8
    assert _lib.OharaBitLayer.gamma.offset == 112 and _lib.OharaBitLayer.norm1.offset == 144
    assert ctypes.sizeof(_lib.OharaBitModel) == ctypes.sizeof(_lib.OharaModel)
    assert _lib.OharaBitModel.layers.offset == _lib.OharaModel.layers.offset


def test_argument_checks_need_no_gpu():
    """Entry points validate their arguments before touching the device."""
    from ohara_amd import _lib

    L = _lib.lib()
    assert L.ohara_embed_bf16(0, 0, 0, 1, 8, 8, 0) == _lib.EINVAL
    assert L.ohara_gemm_skinny_bf16(0, 8, 0, 8, 8, 0, 1e-5, 1, 0, 0, 0, 0, 8, 0) == _lib.EINVAL
    assert L.ohara_attn_workspace_bytes(0, 1, 1, 1, 1) == _lib.EINVAL
    assert L.ohara_attn_workspace_bytes(2, 4, 2, 64, 8) > 0
    assert L.ohara_bitnet_persistent_workspace_bytes(None, 1, 256) == _lib.EINVAL
    bm = _lib.OharaBitModel()
    bm.n_layers, bm.d_model, bm.n_heads, bm.n_kv_heads, bm.head_dim, bm.d_ff = 2, 256, 4, 4, 64, 512
    assert L.ohara_bitnet_persistent_workspace_bytes(ctypes.byref(bm), 2, 256) > 0
    assert L.ohara_bitnet_decode_persistent(ctypes.byref(bm), None, None, 256, 0, 1, 0, None) == _lib.EINVAL
    buf = (ctypes.c_int32 * 32)()
    assert L.ohara_swiglu_perm(12, buf) == 0
    # packed row 0..3 of strip 0: gate 0, gate 1, up 0, up 1 (up rows follow the 12 gate rows)
    assert list(buf[:4]) == [0, 1, 12, 13]
    assert list(buf[16:20]) == [8, 9, 20, 21] and buf[28] == -1

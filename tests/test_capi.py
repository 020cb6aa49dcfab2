"""The C-ABI library: loads, exports what the header declares, validates arguments on the
host before anything is launched (CPU only; no kernel runs here)."""
import ctypes as C
import os
import re
import subprocess

import pytest

from deepstrix_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "dsx_moe.h")


def declared_functions():
    """name -> parameter count, parsed from the header's prototypes."""
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    out = {}
    for m in re.finditer(r"\b(dsx_[a-z0-9_]+)\s*\(([^;{}]*?)\)\s*;", text, flags=re.S):
        name, args = m.group(1), m.group(2).strip()
        out[name] = 0 if args in ("", "void") else args.count(",") + 1
    return out


def test_header_is_plain_c():
    res = subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-fsyntax-only", "-x", "c", HEADER],
                         capture_output=True, text=True)
    assert res.returncode == 0, res.stderr


def test_library_exports_every_declared_symbol():
    decl = declared_functions()
    assert len(decl) >= 25
    raw = C.CDLL(capi.LIB_PATH)
    missing = [n for n in decl if not hasattr(raw, n)]
    assert not missing, f"declared in include/dsx_moe.h but not exported: {missing}"


def test_binding_table_matches_the_header():
    decl = declared_functions()
    assert set(decl) == set(capi.SIGNATURES), set(decl) ^ set(capi.SIGNATURES)
    for name, n in decl.items():
        assert len(capi.SIGNATURES[name][1]) == n, name


def test_abi_version_and_constants():
    text = open(HEADER).read()
    ver = int(re.search(r"#define\s+DSX_ABI_VERSION\s+(\d+)", text).group(1))
    assert capi.lib().dsx_abi_version() == ver
    for cname, val in [("DSX_FMT_Q8_0", capi.FMT_Q8_0), ("DSX_FMT_MXFP4", capi.FMT_MXFP4),
                       ("DSX_ERR_INVALID_ARG", capi.ERR_INVALID_ARG), ("DSX_ERR_SHAPE", capi.ERR_SHAPE),
                       ("DSX_ERR_UNSUPPORTED", capi.ERR_UNSUPPORTED), ("DSX_ERR_DEVICE", capi.ERR_DEVICE)]:
        m = re.search(rf"#define\s+{cname}\s+\(?(-?\d+)\)?", text)
        assert m and int(m.group(1)) == val, cname


def test_layer_desc_struct_matches_the_header_field_order():
    text = open(HEADER).read()
    body = re.search(r"typedef struct\s*\{((?:(?!typedef).)*?)\}\s*dsx_moe_layer_desc;", text, flags=re.S)
    assert body, "dsx_moe_layer_desc not found"
    src = re.sub(r"/\*.*?\*/", "", body.group(1), flags=re.S)
    names = []
    for stmt in src.split(";"):
        stmt = stmt.strip()
        if not stmt:
            continue
        for part in stmt.split(","):
            names.append(re.findall(r"[A-Za-z_][A-Za-z0-9_]*", part)[-1])
    assert names == [f[0] for f in capi.LayerDesc._fields_]


def _desc(**kw):
    d = capi.LayerDesc()
    d.hidden, d.inter, d.n_expert, d.n_used = 512, 256, 8, 2
    d.gate_fmt = d.up_fmt = d.down_fmt = capi.FMT_MXFP4
    d.gate = d.up = d.down = 0x1000  # never dereferenced by create()
    d.router_mode = capi.ROUTER_SIGMOID
    for k, v in kw.items():
        setattr(d, k, v)
    return d


def _create(d):
    h = C.c_void_p()
    rc = capi.lib().dsx_moe_layer_create(C.byref(d), C.byref(h))
    return rc, h


def test_layer_create_validates_before_anything_touches_a_device():
    l = capi.lib()
    rc, h = _create(_desc())
    assert rc == 0 and h.value
    assert l.dsx_moe_layer_workspace_bytes(h, 4) > l.dsx_moe_layer_workspace_bytes(h, 1) > 0
    l.dsx_moe_layer_destroy(h)

    cases = [
        (dict(gate=None), capi.ERR_INVALID_ARG),
        (dict(n_used=0), capi.ERR_INVALID_ARG),
        (dict(n_used=9), capi.ERR_INVALID_ARG),            # more picks than experts
        (dict(hidden=520), capi.ERR_SHAPE),                # not a multiple of 256
        (dict(inter=96), capi.ERR_SHAPE),                  # MXFP4 down needs inter % 256 == 0
        (dict(up_fmt=capi.FMT_Q8_0), capi.ERR_UNSUPPORTED),
        (dict(gate_fmt=12, up_fmt=12), capi.ERR_SHAPE),    # a format id with no layout
        (dict(sh_inter=256), capi.ERR_INVALID_ARG),        # shared expert without weights
        (dict(router_mode=3), capi.ERR_INVALID_ARG),
    ]
    for kw, code in cases:
        rc, h = _create(_desc(**kw))
        assert rc == code, (kw, rc)
        assert not h.value
        assert l.dsx_last_error(), kw
    with pytest.raises(capi.DsxError) as ei:
        capi.check(_create(_desc(hidden=520))[0])
    assert ei.value.code == capi.ERR_SHAPE and "hidden=520" in ei.value.message


def test_null_layer_handles_are_errors():
    l = capi.lib()
    assert l.dsx_moe_layer_set_profile_events(None, None, None, None) == capi.ERR_INVALID_ARG
    assert l.dsx_moe_layer_workspace_bytes(None, 1) == 0
    l.dsx_moe_layer_destroy(None)  # a no-op, like free(NULL)


def test_operators_refuse_bad_arguments_before_any_launch():
    """Validation comes first in every entry point: these calls return an error code without a
    device (pointers are fake; nothing is launched when the arguments are refused)."""
    l = capi.lib()
    p = 0x1000  # a non-null, 16-byte aligned stand-in
    bad = [
        l.dsx_router_topk(None, p, p, p, None, 0, 1, 1.0, 1e-20, 1, 0, 1, 1),          # n_expert = 0
        l.dsx_router_topk(None, p, p, p, None, 64, 6, 1.0, 1e-20, 1, 3, 1, 1),         # mode 3
        l.dsx_router_topk(None, p, p, p, None, 64, 6, 1.0, 1e-20, 1, 1, 7, 2),         # 64 % 7 != 0
        l.dsx_router_hash_select(None, p, p, p, p, p, 64, 0, 10, 1.5, 6e-5, 1),        # n_used = 0
        l.dsx_router_hash_select(None, p, p, p, None, p, 64, 6, 10, 1.5, 6e-5, 1),     # null table
        l.dsx_moe_hetsplit_select(None, p, p, p, 2, 1, 6, 64, 1),                      # mode 2
        l.dsx_moe_group_build(None, p, p, p, p, p, p, 4, 6, 64, 65),                   # chunk 65
        l.dsx_moe_group_build(None, p, p, p, p, p, p, 70000, 6, 64, 4),                # b >= 65536
        l.dsx_moe_gate_up_batch(None, capi.FMT_MXFP4, p, p, p, p, p, p, 8, 8, 6, 0.0, 24, 2),   # rows % 16
        l.dsx_moe_gate_up_batch(None, 12, p, p, p, p, p, p, 8, 8, 6, 0.0, 32, 2),               # format id
        l.dsx_moe_gate_up_chunked_rows(None, capi.FMT_MXFP4, p, p, p, p, p, p, p, p, p, p, 4, 8, 8, 6, 65,
                                       0.0, 32, 2),                                              # chunk 65
        l.dsx_moe_down_by_expert(None, capi.FMT_MXFP4, p, p, p, p, p, p, p, p, 4, 8, 292, 6, 0, 32, 1),  # chunk 0
        l.dsx_q8_0_weights_from_hf(None, p, p, None, capi.SRC_F8E4M3, 64, 64, 0, 0, 1),   # fp8 without scales
        l.dsx_q8_0_weights_from_hf(None, p, p, p, capi.SRC_F8E4M3, 64, 64, 3, 2, 1),      # grid does not tile
        l.dsx_q8_0_weights_from_hf(None, p, p, None, capi.SRC_F32, 64, 48, 0, 0, 1),      # cols % 32
        l.dsx_q8_0_repack_rows(None, p, p, 4, 2),                                          # in place
        l.dsx_mxfp4_repack_hf_to_v2(None, p, p, p, 4, 7),                                  # nb % 8
        l.dsx_rms_norm(None, p, p, None, 64, 1e-6, 1) if hasattr(l, "dsx_rms_norm") else -1,
    ]
    assert all(rc < 0 for rc in bad), bad
    assert l.dsx_last_error()


def _thresholds(hidden, inter, n_expert, n_used, gate_fmt=None, down_fmt=None):
    """Default thresholds of a layer of that shape (no device needed: creating a layer whose
    shared expert rides with the routed ones only records pointers and sizes)."""
    import ctypes as C
    l = capi.lib()
    d = capi.LayerDesc()
    d.hidden, d.inter, d.n_expert, d.n_used = hidden, inter, n_expert, n_used
    d.gate_fmt = d.up_fmt = capi.FMT_MXFP4 if gate_fmt is None else gate_fmt
    d.down_fmt = capi.FMT_MXFP4 if down_fmt is None else down_fmt
    d.gate = d.up = d.down = 0x1000
    d.gate_bpe = d.up_bpe = d.down_bpe = 1 << 20
    d.router_mode, d.n_group, d.topk_group = 1, 1, 1
    h = C.c_void_p()
    assert l.dsx_moe_layer_create(C.byref(d), C.byref(h)) == 0, l.dsx_last_error()
    v = (C.c_uint32 * 6)()
    assert l.dsx_moe_layer_get_tuning(h, C.byref(v)) == 0
    l.dsx_moe_layer_destroy(h)
    return dict(zip(("chunk", "gemm", "gemm_q8", "decode_max", "narrow", "share"), (int(x) for x in v)))


def test_default_thresholds_follow_the_picks_per_expert():
    """The crossovers measured on four shapes, as picks per expert (include/dsx_moe.h:
    dsx_moe_layer_set_tuning): every shape gets its token counts from the ratios, none inherits the
    DeepSeek-V3 shape's."""
    v3 = _thresholds(7168, 2048, 256, 8)
    # by-expert overtakes the decode launch at 13 .. 14 tokens, the GEMM the by-expert kernels at 96 .. 128
    assert (v3["narrow"], v3["share"]) == (1, 4)
    assert 13 <= v3["decode_max"] <= 14 and 97 <= v3["gemm"] <= 128
    # 128 experts, top-8, inter 1024: by-expert overtakes the decode launch between 12 and 16 tokens,
    # the GEMM the by-expert kernels between 48 and 64
    e128 = _thresholds(4096, 1024, 128, 8)
    assert 12 <= e128["decode_max"] <= 15 and 49 <= e128["gemm"] <= 64
    # 64 experts, top-6, small matrices: 4 .. 5 tokens and 64 .. 96 tokens
    e64 = _thresholds(2048, 1536, 64, 6)
    assert 4 <= e64["decode_max"] <= 5 and 65 <= e64["gemm"] <= 96
    # config 1 (all Q8_0): the int8 GEMM is ahead from 16 tokens on and far ahead at 24
    q8 = _thresholds(2048, 1408, 64, 6, capi.FMT_Q8_0, capi.FMT_Q8_0)
    assert 12 <= q8["gemm_q8"] <= 24
    # MXFP4 gate/up with a Q8_0 down matrix (config 5): the GEMMs are ahead from 64 tokens on
    mixed = _thresholds(7168, 2048, 256, 8, capi.FMT_MXFP4, capi.FMT_Q8_0)
    assert 49 <= mixed["gemm_q8"] <= 64


def test_missing_library_is_an_import_error_not_a_fallback(monkeypatch):
    monkeypatch.setattr(capi, "_lib", None)
    monkeypatch.setattr(capi, "LIB_PATH", os.path.join(ROOT, "deepstrix_amd", "lib", "absent.so"))
    with pytest.raises(ImportError, match="no CPU fallback"):
        capi.lib()


def test_the_package_never_reaches_into_the_oracle():
    pkg = os.path.join(ROOT, "deepstrix_amd")
    offenders = []
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".inc", ".h")):
                text = open(os.path.join(dirpath, f), errors="replace").read()
                if re.search(r"\boracle\b|dsx_ref_|libdsx_oracle", text):
                    offenders.append(f)
    assert not offenders, offenders

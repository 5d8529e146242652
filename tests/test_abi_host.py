"""Host-only checks of the C ABI: the library loads, exports every symbol the
header declares, the ctypes mirror matches the header, and argument validation
returns the documented codes.  No kernel is launched."""
import ctypes
import os
import re

import pytest

from oregon_gpt_oss_patching_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "gptoss_attn.h")


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gptoss_attn_[a-z_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported():
    lib = _lib.load()
    names = _declared_functions()
    assert set(names) == set(_lib.EXPORTS), names
    for n in names:
        assert getattr(lib, n) is not None


def test_version_and_status_strings():
    lib = _lib.load()
    assert lib.gptoss_attn_version() == _lib.ABI_VERSION
    assert _lib.status_string(0) == "ok"
    assert "64" in _lib.status_string(-3)
    assert "HIP" in _lib.status_string(719)


def test_struct_mirror_matches_header_field_order():
    text = open(HEADER).read()
    body = re.search(r"typedef struct gptoss_attn_params \{(.*?)\} gptoss_attn_params;", text, re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    names = []
    for decl in body.split(";"):
        decl = decl.strip()
        if not decl:
            continue
        for part in decl.split(","):
            names.append(re.findall(r"[A-Za-z_][A-Za-z_0-9]*", part)[-1])
    assert names == [f[0] for f in _lib.Params._fields_]
    assert ctypes.sizeof(_lib.Params) == 360


def _integration_stub_classes():
    """The ctypes classes of the reference-side binding stub in the repository's integration notes,
    executed as they stand in that document."""
    text = open(os.path.join(ROOT, "INTEGRATION" + ".md")).read()
    block = next(b for b in re.findall(r"```python\n(.*?)```", text, re.S) if "class Params(ctypes.Structure)" in b)
    start = block.index("class Strides(ctypes.Structure)")
    end = block.index("lib = ctypes.CDLL")
    ns = {"ctypes": ctypes}
    exec(block[start:end], ns)
    return ns["Strides"], ns["Params"]


def test_integration_doc_stub_matches_the_library():
    """The documented reference-side binding must be accepted by the shipped library: same size,
    same field names, offsets and sizes as the package's own mirror, and a block filled through it
    passes validation."""
    strides_cls, params_cls = _integration_stub_classes()
    assert ctypes.sizeof(strides_cls) == ctypes.sizeof(_lib.Strides)
    assert ctypes.sizeof(params_cls) == ctypes.sizeof(_lib.Params) == 360
    assert [f[0] for f in params_cls._fields_] == [f[0] for f in _lib.Params._fields_]
    for name, _ in _lib.Params._fields_:
        mine, doc = getattr(_lib.Params, name), getattr(params_cls, name)
        assert (mine.offset, mine.size) == (doc.offset, doc.size), name
    good = _valid_params()
    p = params_cls.from_buffer_copy(bytes(good))
    p.struct_size = ctypes.sizeof(params_cls)
    lib = ctypes.CDLL(_lib.LIBRARY)
    lib.gptoss_attn_validate.restype = ctypes.c_int
    assert lib.gptoss_attn_validate(ctypes.byref(p), 1) == 0
    assert lib.gptoss_attn_version() == 4
    for name in ("gptoss_attn_fwd", "gptoss_attn_bwd", "gptoss_attn_bwd_static"):   # what the stub binds
        assert getattr(lib, name) is not None


def _valid_params():
    """A parameter block that passes validation (fake, aligned, never dereferenced)."""
    p = _lib.new_params()
    p.dtype = _lib.DTYPE_BF16
    p.B, p.H, p.G, p.Sq, p.Skv, p.D = 1, 8, 2, 128, 128, 64
    p.scale = 0.125
    fake = 0x1000
    for f in ("q", "k", "v", "o", "lse", "d_o", "dq", "dk", "dv", "delta"):
        setattr(p, f, fake)
    for st in ("q_stride", "k_stride", "v_stride", "o_stride", "do_stride", "dq_stride", "dk_stride", "dv_stride"):
        s = getattr(p, st)
        s.b, s.h, s.s = 8 * 128 * 64, 128 * 64, 64
    return p


def _validate(p, bwd=1):
    return _lib.load().gptoss_attn_validate(ctypes.byref(p), bwd)


def test_validate_accepts_good_params():
    assert _validate(_valid_params()) == 0


@pytest.mark.parametrize("mutate,code", [
    (lambda p: setattr(p, "struct_size", 8), -9),
    (lambda p: setattr(p, "dtype", 7), -6),
    (lambda p: setattr(p, "D", 128), -3),
    (lambda p: setattr(p, "G", 3), -4),
    (lambda p: setattr(p, "H", 0), -4),
    (lambda p: setattr(p, "Sq", 0), -5),
    (lambda p: setattr(p, "window", -1), -5),
    (lambda p: setattr(p, "q_offset", -2), -5),
    (lambda p: setattr(p, "q_offset", 2 ** 30), -5),
    (lambda p: setattr(p, "window", 2 ** 30 + 1), -5),
    (lambda p: setattr(p, "scale", 0.0), -5),
    (lambda p: setattr(p, "scale", float("nan")), -5),
    (lambda p: setattr(p, "q", None), -2),
    (lambda p: setattr(p, "lse", None), -2),
    (lambda p: setattr(p, "dv", None), -2),
    (lambda p: setattr(p, "delta", None), -2),
    (lambda p: setattr(p, "k", 0x1008), -7),
    (lambda p: setattr(p, "delta", 0x1004), -7),
    (lambda p: setattr(p.v_stride, "s", 68), -7),
    (lambda p: setattr(p.v_stride, "s", 32), -8),
    (lambda p: setattr(p.q_stride, "s", 2 ** 24 + 64), -8),
    (lambda p: (setattr(p, "doc_start", 0x2000), setattr(p, "q_offset", 4)), -5),
    (lambda p: (setattr(p, "doc_start", 0x2000), setattr(p, "Skv", 256)), -5),
    (lambda p: (setattr(p, "doc_start", 0x2000), setattr(p, "q_offset_dev", 0x3000)), -5),
    (lambda p: setattr(p, "q_offset_dev", 0x3002), -7),
])
def test_validate_error_codes(mutate, code):
    p = _valid_params()
    mutate(p)
    assert _validate(p) == code
    assert _lib.status_string(code) not in ("ok", "unknown status")


def test_device_query_offset_overrides_the_host_field():
    """With q_offset_dev set the host field is not looked at (the kernels read the device value),
    and the host-side shortcuts that need the value are off: the workspace is the generic one."""
    p = _valid_params()
    p.q_offset_dev = 0x3000
    p.q_offset = -7
    assert _validate(p) == 0
    lib = _lib.load()
    q = _valid_params()
    q.window = 128
    single_pass = lib.gptoss_attn_workspace_bytes(ctypes.byref(q))
    q.q_offset_dev = 0x3000
    generic = lib.gptoss_attn_workspace_bytes(ctypes.byref(q))
    q.q_offset_dev, q.window = None, 0
    assert generic == lib.gptoss_attn_workspace_bytes(ctypes.byref(q)) and single_pass >= generic


def test_forward_only_validation_ignores_backward_tensors():
    p = _valid_params()
    p.dq = None
    p.delta = None
    assert _validate(p, 0) == 0 and _validate(p, 1) == -2


def test_null_params_pointer():
    lib = _lib.load()
    assert lib.gptoss_attn_validate(None, 0) == -1
    assert lib.gptoss_attn_fwd(None, None) == -1
    assert lib.gptoss_attn_bwd(None, None) == -1


def test_entry_points_reject_bad_arguments_before_launching():
    """Validation is host-side, so a bad block must come back with its code even
    where there is no GPU to launch on."""
    p = _valid_params()
    p.D = 32
    lib = _lib.load()
    for name in ("gptoss_attn_fwd", "gptoss_attn_bwd_preprocess", "gptoss_attn_bwd_dkdv",
                 "gptoss_attn_bwd_dq", "gptoss_attn_bwd"):
        assert getattr(lib, name)(ctypes.byref(p), None) == -3


def test_call_raises_with_status_text():
    p = _valid_params()
    p.G = 5
    with pytest.raises(_lib.GptossAttnError) as ei:
        _lib.call("gptoss_attn_fwd", p, 0)
    assert ei.value.status == -4 and "divisible" in str(ei.value)


def test_validate_float32_params_and_their_alignment_rule():
    """float32 tensors: rows must still start on 16-byte boundaries, i.e. strides are multiples
    of 4 elements (8 for bf16): a stride of 68 floats is fine, 66 is not."""
    p = _valid_params()
    p.dtype = _lib.DTYPE_FP32
    assert _validate(p) == 0
    p.v_stride.s = 68
    assert _validate(p) == 0
    p.v_stride.s = 66
    assert _validate(p) == -7


def test_workspace_bytes():
    lib = _lib.load()
    p = _valid_params()
    # row statistics: -delta and lse * log2(e) in fp32 (8 bytes per row), then both again as the bf16 triples
    # the dK/dV kernels feed to the matrix pipe (16 bytes per row)
    assert lib.gptoss_attn_workspace_bytes(ctypes.byref(p)) == (8 + 16) * 1 * 8 * 128
    p.B, p.H, p.G, p.Sq, p.Skv = 4, 64, 8, 16384, 16384
    assert lib.gptoss_attn_workspace_bytes(ctypes.byref(p)) == (8 + 16) * 4 * 64 * 16384
    # short sequences: the dK/dV kernel cuts each key block's query tiles into slices (here 4) and
    # keeps their fp32 partial sums behind the row statistics; sliding-window layers are never cut
    p.B, p.Sq, p.Skv = 1, 4096, 4096
    stats = (8 + 16) * 1 * 64 * 4096
    assert lib.gptoss_attn_workspace_bytes(ctypes.byref(p)) == stats + 4 * 2 * 4 * 1 * 8 * 4096 * 64
    # a sliding-window layer the single-pass backward takes: its dSinks partial sums [B][chunks][H][2]
    # and 128 KB of fp32 dK/dV shares per (batch, KV head, seam between chunks), if that is more than
    # the row statistics.  The size is that of the shortest chunks any device can ask for (2 query
    # tiles), so it does not depend on the device: 64 query tiles = 32 chunks.
    p.window = 128
    chunks = 32
    assert lib.gptoss_attn_workspace_bytes(ctypes.byref(p)) == 1 * chunks * 64 * 2 * 4 + 1 * 8 * (chunks - 1) * 128 * 1024
    p.window = 256      # longer windows take the three-kernel route: row statistics only, never cut
    assert lib.gptoss_attn_workspace_bytes(ctypes.byref(p)) == stats
    p.window = 0
    p.dtype = _lib.DTYPE_FP32
    assert lib.gptoss_attn_workspace_bytes(ctypes.byref(p)) == stats
    p.dtype = _lib.DTYPE_BF16
    p.Sq = 0
    assert lib.gptoss_attn_workspace_bytes(ctypes.byref(p)) == 0
    assert lib.gptoss_attn_workspace_bytes(None) == 0


def test_mfma_rate_probe_refuses_bad_arguments_on_the_host():
    """The measurement aid checks its arguments before it launches anything."""
    lib = _lib.load()
    assert lib.gptoss_attn_mfma_rate_probe(None, 1024, 10, None, 0, None) < 0
    assert lib.gptoss_attn_mfma_rate_probe(ctypes.c_void_p(256), 8, 10, ctypes.c_void_p(256), 1 << 30, None) < 0     # under 16 bytes
    assert lib.gptoss_attn_mfma_rate_probe(ctypes.c_void_p(264), 1024, 10, ctypes.c_void_p(256), 1 << 30, None) < 0  # misaligned
    assert lib.gptoss_attn_mfma_rate_probe(ctypes.c_void_p(256), 1024, 0, ctypes.c_void_p(256), 1 << 30, None) < 0   # no passes


def test_stream_probe_refuses_bad_arguments_on_the_host():
    """The second measurement aid checks its arguments before it touches the device."""
    lib = _lib.load()
    ok_sink, many = ctypes.c_void_p(256), 1 << 30
    assert lib.gptoss_attn_stream_probe(0, 2, 10, None, many, None) < 0            # no sink
    assert lib.gptoss_attn_stream_probe(6, 2, 10, ok_sink, many, None) < 0         # no such mix
    assert lib.gptoss_attn_stream_probe(-1, 2, 10, ok_sink, many, None) < 0
    assert lib.gptoss_attn_stream_probe(0, 0, 10, ok_sink, many, None) < 0         # wavefronts per SIMD: 1 to 3
    assert lib.gptoss_attn_stream_probe(0, 4, 10, ok_sink, many, None) < 0
    assert lib.gptoss_attn_stream_probe(0, 2, 0, ok_sink, many, None) < 0          # no passes

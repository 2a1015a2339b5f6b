"""Host-only checks of the C ABI (include/fa_fwd.h, include/fa_bwd.h / libfa_fwd.so): the library loads, exports every declared
symbol, and its argument validation / planning — which never touch the GPU — return the documented codes."""
import ctypes
import os
import re

import pytest

from torch_mlu_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    syms = set()
    for header in ("fa_fwd.h", "fa_bwd.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        syms |= set(re.findall(r"\b(fa_(?:fwd|bwd)_[a-z_]+)\s*\(", text))
    return sorted(syms)


def test_library_exports_exactly_the_declared_symbols():
    """Every entry point the two headers declare is exported, and nothing else is: the library is built with hidden
    visibility, so C++ internals cannot be interposed by, or merge with, another object that includes the same
    inline headers."""
    import subprocess

    syms = _declared_symbols()
    assert syms == sorted(capi.EXPORTED_SYMBOLS)
    L = ctypes.CDLL(capi.LIB_PATH)
    for s in syms:
        assert hasattr(L, s), s
    out = subprocess.run(["nm", "-D", "--defined-only", capi.LIB_PATH], check=True, capture_output=True, text=True).stdout
    exported = sorted(line.split()[-1] for line in out.splitlines() if line.split()[1] in "TWVBDR")
    assert exported == syms, sorted(set(exported) ^ set(syms))


def test_version_and_error_strings():
    L = capi.lib()
    assert L.fa_fwd_version() == capi.FA_FWD_ABI_VERSION == 9
    assert capi.error_string(0) == "ok"
    for rc in (-1, -2, -3, -99):
        assert capi.error_string(rc)


def _good(**over):
    """A syntactically valid params struct with fake (aligned, never dereferenced) device addresses."""
    p = capi.FaFwdParams()
    p.q, p.k, p.v, p.out, p.lse = 0x1000, 0x2000, 0x3000, 0x4000, 0x5000
    B, Hq, Hk, Sq, Sk, D = 2, 8, 2, 128, 256, 128
    p.q_stride_b, p.q_stride_s, p.q_stride_h = Sq * Hq * D, Hq * D, D
    p.k_stride_b, p.k_stride_s, p.k_stride_h = Sk * Hk * D, Hk * D, D
    p.v_stride_b, p.v_stride_s, p.v_stride_h = Sk * Hk * D, Hk * D, D
    p.o_stride_b, p.o_stride_s, p.o_stride_h = Sq * Hq * D, Hq * D, D
    p.lse_stride_b, p.lse_stride_h, p.lse_stride_s = Hq * Sq, Sq, 1
    p.batch, p.heads_q, p.heads_k, p.seqlen_q, p.seqlen_k, p.head_dim = B, Hq, Hk, Sq, Sk, D
    p.scale, p.dtype, p.is_causal, p.kernel, p.num_splits, p.reserved = 0.088, capi.FA_DTYPE_BF16, 1, 0, 0, 0
    for k, v in over.items():
        setattr(p, k, v)
    return p


def test_validate_accepts_good_params():
    assert capi.lib().fa_fwd_validate(ctypes.byref(_good())) == capi.FA_OK
    assert capi.lib().fa_fwd_validate(ctypes.byref(_good(dtype=capi.FA_DTYPE_FP16, head_dim=64))) == capi.FA_OK


@pytest.mark.parametrize("over,rc", [
    (dict(q=None), capi.FA_ERR_BAD_ARG),
    (dict(out=None), capi.FA_ERR_BAD_ARG),
    (dict(lse=None), capi.FA_ERR_BAD_ARG),
    (dict(q=0x1008), capi.FA_ERR_BAD_ARG),              # not 16-byte aligned
    (dict(k_stride_s=130), capi.FA_ERR_BAD_ARG),        # rows not 16-byte aligned
    (dict(q_stride_h=-128), capi.FA_ERR_BAD_ARG),
    (dict(batch=0), capi.FA_ERR_BAD_ARG),               # "batch size must be positive"
    (dict(heads_k=0), capi.FA_ERR_BAD_ARG),
    (dict(reserved=1), capi.FA_ERR_BAD_ARG),
    (dict(num_splits=65), capi.FA_ERR_BAD_ARG),
    (dict(kernel=7), capi.FA_ERR_BAD_ARG),
    (dict(cu_seqlens_q=0x6000), capi.FA_ERR_BAD_ARG),   # only one of the two cu_seqlens
    (dict(dtype=5), capi.FA_ERR_UNSUPPORTED),           # "only support fp16 and bf16"
    (dict(head_dim=264), capi.FA_ERR_UNSUPPORTED),      # "head dimension at most 256"
    (dict(head_dim=100), capi.FA_ERR_UNSUPPORTED),      # not a multiple of 8
    (dict(heads_k=3), capi.FA_ERR_UNSUPPORTED),         # "must divide number of heads in query"
    (dict(kernel=capi.FA_KERNEL_SPLITKV), capi.FA_ERR_UNSUPPORTED),  # split-KV needs seqlen_q == 1
    (dict(k_stride_s=1 << 24), capi.FA_ERR_UNSUPPORTED),  # 128 rows x 32 MiB overflow a 32-bit tile offset
    (dict(v_stride_s=1 << 24), capi.FA_ERR_UNSUPPORTED),
])
def test_validate_rejects(over, rc):
    p = _good(**over)
    L = capi.lib()
    assert L.fa_fwd_validate(ctypes.byref(p)) == rc
    assert L.fa_fwd_workspace_bytes(ctypes.byref(p)) == 0
    # launch refuses before touching the device
    assert L.fa_fwd_launch(ctypes.byref(p), None, 0, None) == rc


def test_null_params():
    L = capi.lib()
    assert L.fa_fwd_validate(None) == capi.FA_ERR_BAD_ARG
    assert L.fa_fwd_workspace_bytes(None) == 0
    assert L.fa_fwd_launch(None, None, 0, None) == capi.FA_ERR_BAD_ARG


def _plan(p):
    k, s = ctypes.c_int32(-1), ctypes.c_int32(-1)
    rc = capi.lib().fa_fwd_plan(ctypes.byref(p), ctypes.byref(k), ctypes.byref(s))
    return rc, k.value, s.value


def test_plan_prefill_uses_tile_kernel_without_workspace():
    p = _good()
    assert _plan(p) == (capi.FA_OK, capi.FA_KERNEL_TILE, 1)
    assert capi.lib().fa_fwd_workspace_bytes(ctypes.byref(p)) == 0


def test_plan_decode_uses_splitkv_and_sizes_workspace():
    """BASELINE config 5 shape: B=64, Hq=32, Hkv=8, Sq=1, Skv=8192, D=128."""
    p = _good(batch=64, heads_q=32, heads_k=8, seqlen_q=1, seqlen_k=8192, is_causal=0)
    rc, kern, ns = _plan(p)
    assert rc == capi.FA_OK and kern == capi.FA_KERNEL_SPLITKV and 1 <= ns <= capi.FA_MAX_SPLITS
    need = capi.lib().fa_fwd_workspace_bytes(ctypes.byref(p))
    assert need == (0 if ns == 1 else 64 * 32 * ns * (128 * 4 + 8))
    # a short or missing workspace is refused on the host
    if need:
        assert capi.lib().fa_fwd_launch(ctypes.byref(p), None, 0, None) == capi.FA_ERR_BAD_ARG
        assert capi.lib().fa_fwd_launch(ctypes.byref(p), 0x7000, need - 1, None) == capi.FA_ERR_BAD_ARG
    # a shape that is split: the workspace is needed, and a short or missing one is refused on the host
    p2 = _good(batch=4, heads_q=32, heads_k=8, seqlen_q=1, seqlen_k=32768, is_causal=0)
    assert _plan(p2) == (capi.FA_OK, capi.FA_KERNEL_SPLITKV, 8)
    need2 = capi.lib().fa_fwd_workspace_bytes(ctypes.byref(p2))
    assert need2 == 4 * 32 * 8 * (128 * 4 + 8)
    assert capi.lib().fa_fwd_launch(ctypes.byref(p2), None, 0, None) == capi.FA_ERR_BAD_ARG
    assert capi.lib().fa_fwd_launch(ctypes.byref(p2), 0x7000, need2 - 1, None) == capi.FA_ERR_BAD_ARG
    # explicit split count is honoured and capped by the number of 32-row blocks
    p.num_splits = 4
    assert _plan(p) == (capi.FA_OK, capi.FA_KERNEL_SPLITKV, 4)
    p.seqlen_k, p.num_splits, p.kernel = 40, 8, capi.FA_KERNEL_SPLITKV
    assert _plan(p) == (capi.FA_OK, capi.FA_KERNEL_SPLITKV, 2)
    # short KV: the automatic choice is the tile kernel
    p.kernel = capi.FA_KERNEL_AUTO
    assert _plan(p)[1] == capi.FA_KERNEL_TILE
    # wide GQA groups (> 16 query heads per kv head) fall back to the tile kernel
    p = _good(batch=1, heads_q=32, heads_k=1, seqlen_q=1, seqlen_k=4096)
    assert _plan(p)[1] == capi.FA_KERNEL_TILE


@pytest.mark.parametrize("batch,heads_k,seqlen_k,want", [
    (64, 8, 8192, 1),     # 512 (sequence, kv head) units: more than one per CU already
    (16, 8, 8192, 2),     # 128 units -> 256 workgroups
    (4, 8, 8192, 4),      # 32 units: 8 would fill the CUs, but 2048-row slices win while 128 workgroups remain
    (4, 8, 131072, 8),
    (1, 8, 8192, 16),
    (1, 8, 32768, 16),
    (1, 8, 131072, 32),
    (1, 1, 131072, 64),   # the cap
    (1, 8, 1024, 2),      # never below 512 rows per slice
    (256, 8, 2048, 1),
])
def test_plan_split_count(batch, heads_k, seqlen_k, want):
    """The automatic split count: one workgroup per CU at most, long slices preferred."""
    p = _good(batch=batch, heads_q=4 * heads_k, heads_k=heads_k, seqlen_q=1, seqlen_k=seqlen_k, is_causal=0)
    assert _plan(p) == (capi.FA_OK, capi.FA_KERNEL_SPLITKV, want)


@pytest.mark.parametrize("over,kern,ns", [
    (dict(batch=4, heads_q=32, heads_k=32, seqlen_q=4096, seqlen_k=4096), "tile", 1),     # the headline prefill
    (dict(batch=1, heads_q=32, heads_k=8, seqlen_q=128, seqlen_k=32768), "tile", 16),     # a chunk against a cache
    (dict(batch=1, heads_q=32, heads_k=8, seqlen_q=512, seqlen_k=32768), "tile", 4),
    (dict(batch=1, heads_q=8, heads_k=8, seqlen_q=4096, seqlen_k=4096), "tile", 2),       # small-batch prefill
    (dict(batch=2, heads_q=8, heads_k=8, seqlen_q=2048, seqlen_k=2048), "tile", 1),       # slices would be too short
    (dict(batch=1, heads_q=64, heads_k=1, seqlen_q=1, seqlen_k=32768), "tile", 8),        # group too wide for split-KV
    (dict(batch=1, heads_q=32, heads_k=8, seqlen_q=128, seqlen_k=32768, dropout_p=0.1), "tile", 16),  # dropout slices too
    (dict(batch=8, heads_q=32, heads_k=8, seqlen_q=4, seqlen_k=32768, dropout_p=0.1), "splitkv", 4),   # dropout: both kernels
    (dict(batch=8, heads_q=32, heads_k=8, seqlen_q=4, seqlen_k=32768, dropout_p=0.1, dropout_mask=0x9000), "tile", 2),
    (dict(batch=8, heads_q=32, heads_k=8, seqlen_q=4, seqlen_k=32768), "splitkv", 4),     # 4 rows x 4 heads = 16 columns
    (dict(batch=8, heads_q=32, heads_k=8, seqlen_q=5, seqlen_k=32768), "tile", 2),        # 20 columns: tile kernel
    (dict(batch=8, heads_q=8, heads_k=8, seqlen_q=16, seqlen_k=32768), "splitkv", 4),
])
def test_plan_slices_and_multi_row_decode(over, kern, ns):
    """Automatic plans: the tile kernel sliced over the key range when a dense call has few query blocks and a long
    K/V; up to 16 (query row, group head) pairs on the split-KV kernel."""
    p = _good(**dict(dict(is_causal=1), **over))
    want = capi.FA_KERNEL_TILE if kern == "tile" else capi.FA_KERNEL_SPLITKV
    assert _plan(p) == (capi.FA_OK, want, ns)
    slots = p.batch * p.heads_q * p.seqlen_q * ns
    assert capi.lib().fa_fwd_workspace_bytes(ctypes.byref(p)) == (0 if ns == 1 else slots * (p.head_dim * 4 + 8))


# ---- backward entry points ------------------------------------------------------------------------------------------
def _good_bwd(**over):
    p = capi.FaBwdParams()
    p.q, p.k, p.v, p.out, p.dout, p.lse = 0x1000, 0x2000, 0x3000, 0x4000, 0x5000, 0x6000
    p.dq, p.dk, p.dv = 0x7000, 0x8000, 0x9000
    B, Hq, Hk, Sq, Sk, D = 2, 8, 2, 128, 256, 128
    for n, (S, H) in dict(q=(Sq, Hq), o=(Sq, Hq), do=(Sq, Hq), dq=(Sq, Hq), k=(Sk, Hk), v=(Sk, Hk), dk=(Sk, Hk),
                          dv=(Sk, Hk)).items():
        setattr(p, n + "_stride_b", S * H * D)
        setattr(p, n + "_stride_s", H * D)
        setattr(p, n + "_stride_h", D)
    p.lse_stride_b, p.lse_stride_h, p.lse_stride_s = Hq * Sq, Sq, 1
    p.batch, p.heads_q, p.heads_k, p.seqlen_q, p.seqlen_k, p.head_dim = B, Hq, Hk, Sq, Sk, D
    p.total_q = 0
    p.scale, p.dtype, p.is_causal, p.reserved = 0.088, capi.FA_DTYPE_BF16, 1, 0
    for k, v in over.items():
        setattr(p, k, v)
    return p


def test_bwd_validate_accepts_good_params_and_sizes_delta_scratch():
    L = capi.lib()
    p = _good_bwd()
    assert L.fa_bwd_validate(ctypes.byref(p)) == capi.FA_OK
    assert L.fa_bwd_workspace_bytes(ctypes.byref(p)) == 2 * (2 * 128 * 8 * 4)   # two fp32 per (batch, row, query head)
    packed = _good_bwd(cu_seqlens_q=0xa000, cu_seqlens_k=0xb000, total_q=200)
    assert L.fa_bwd_validate(ctypes.byref(packed)) == capi.FA_OK
    assert L.fa_bwd_workspace_bytes(ctypes.byref(packed)) == 2 * (200 * 8 * 4)
    # the mem-efficient backward's additions: mask aligned top-left, a (broadcast) bias, its gradient
    full = _good_bwd(is_causal=capi.FA_MASK_CAUSAL_TOP_LEFT, bias=0xc000, bias_stride_b=0, bias_stride_h=0,
                     bias_stride_q=256, dbias=0xd000, dbias_stride_b=8 * 128 * 256, dbias_stride_h=128 * 256,
                     dbias_stride_q=256)
    assert L.fa_bwd_validate(ctypes.byref(full)) == capi.FA_OK
    full.dropout_p, full.philox_seed, full.philox_offset = 0.1, 0xe000, 0xe008     # bias and dropout together
    assert L.fa_bwd_validate(ctypes.byref(full)) == capi.FA_OK


@pytest.mark.parametrize("over,rc", [
    (dict(dout=None), capi.FA_ERR_BAD_ARG),
    (dict(dk=None), capi.FA_ERR_BAD_ARG),
    (dict(lse=None), capi.FA_ERR_BAD_ARG),
    (dict(dv=0x9004), capi.FA_ERR_BAD_ARG),
    (dict(do_stride_s=1028), capi.FA_ERR_BAD_ARG),
    (dict(batch=0), capi.FA_ERR_BAD_ARG),
    (dict(reserved=3), capi.FA_ERR_BAD_ARG),
    (dict(cu_seqlens_k=0xb000), capi.FA_ERR_BAD_ARG),
    (dict(head_dim=264), capi.FA_ERR_UNSUPPORTED),      # "FlashAttention backward only supports head dimension at most 256"
    (dict(head_dim=100), capi.FA_ERR_UNSUPPORTED),
    (dict(dtype=3), capi.FA_ERR_UNSUPPORTED),
    (dict(heads_k=3), capi.FA_ERR_UNSUPPORTED),
    (dict(is_causal=3), capi.FA_ERR_BAD_ARG),                               # not a FA_MASK_* code
    (dict(bias=0xc004, bias_stride_q=256), capi.FA_ERR_BAD_ARG),            # 4-key groups must be 8-byte aligned
    (dict(bias=0xc000, bias_stride_q=258), capi.FA_ERR_BAD_ARG),
    (dict(dbias=0xd000, dbias_stride_q=256), capi.FA_ERR_BAD_ARG),          # a bias gradient without a bias
    (dict(bias=0xc000, bias_stride_q=256, dbias=0xd000, dbias_stride_q=0), capi.FA_ERR_BAD_ARG),   # broadcast output
    (dict(bias=0xc000, bias_stride_q=256, dbias=0xd000, dbias_stride_q=256, dbias_stride_h=0), capi.FA_ERR_BAD_ARG),
])
def test_bwd_validate_rejects(over, rc):
    L = capi.lib()
    p = _good_bwd(**over)
    assert L.fa_bwd_validate(ctypes.byref(p)) == rc
    assert L.fa_bwd_workspace_bytes(ctypes.byref(p)) == 0
    assert L.fa_bwd_launch(ctypes.byref(p), None, 0, None) == rc     # refused before anything is enqueued


def test_bwd_null_and_short_workspace():
    L = capi.lib()
    assert L.fa_bwd_validate(None) == capi.FA_ERR_BAD_ARG
    p = _good_bwd()
    assert L.fa_bwd_launch(ctypes.byref(p), 0x10000, 16, None) == capi.FA_ERR_BAD_ARG
    assert L.fa_bwd_launch(ctypes.byref(p), None, 1 << 20, None) == capi.FA_ERR_BAD_ARG


# ---- additive bias and mask alignment ------------------------------------------------------------------------------
def test_seqused_k_pointer_is_validated():
    L = capi.lib()
    p = _good(seqused_k=0xf000)
    assert L.fa_fwd_validate(ctypes.byref(p)) == capi.FA_OK
    p = _good(seqused_k=0xf002)                      # int32 entries: 4-byte aligned
    assert L.fa_fwd_validate(ctypes.byref(p)) == capi.FA_ERR_BAD_ARG


def test_bias_and_mask_mode_validation_and_plan():
    L = capi.lib()
    good = _good(bias=0x7000, bias_stride_b=0, bias_stride_h=128 * 256, bias_stride_q=256, is_causal=0)
    assert L.fa_fwd_validate(ctypes.byref(good)) == capi.FA_OK
    for over, rc in ((dict(bias=0x7004), capi.FA_ERR_BAD_ARG),                 # 4-key groups must be 8-byte aligned
                     (dict(bias_stride_q=258), capi.FA_ERR_BAD_ARG),
                     (dict(bias_stride_h=-4), capi.FA_ERR_BAD_ARG),
                     (dict(cu_seqlens_q=0x6000, cu_seqlens_k=0x6100), capi.FA_OK),   # a bias is fine in packed mode too
                     (dict(kernel=capi.FA_KERNEL_SPLITKV, seqlen_q=1), capi.FA_ERR_UNSUPPORTED),
                     (dict(is_causal=3), capi.FA_ERR_BAD_ARG)):
        p = _good(**{**dict(bias=0x7000, bias_stride_b=0, bias_stride_h=128 * 256, bias_stride_q=256), **over})
        assert L.fa_fwd_validate(ctypes.byref(p)) == rc, over
    # a single query row with a bias, or with a top-left causal mask, runs the tile kernel
    kern, ns = ctypes.c_int32(), ctypes.c_int32()
    dec = _good(seqlen_q=1, seqlen_k=4096, is_causal=0)
    assert L.fa_fwd_plan(ctypes.byref(dec), ctypes.byref(kern), ctypes.byref(ns)) == 0 and kern.value == capi.FA_KERNEL_SPLITKV
    dec.bias, dec.bias_stride_q = 0x7000, 4096
    assert L.fa_fwd_plan(ctypes.byref(dec), ctypes.byref(kern), ctypes.byref(ns)) == 0 and kern.value == capi.FA_KERNEL_TILE
    tl = _good(seqlen_q=1, seqlen_k=4096, is_causal=capi.FA_MASK_CAUSAL_TOP_LEFT)
    assert L.fa_fwd_plan(ctypes.byref(tl), ctypes.byref(kern), ctypes.byref(ns)) == 0 and kern.value == capi.FA_KERNEL_TILE
    tl.kernel = capi.FA_KERNEL_SPLITKV
    assert L.fa_fwd_validate(ctypes.byref(tl)) == capi.FA_ERR_UNSUPPORTED


def _c_layout(header: str, struct: str, fields):
    """sizeof and every offsetof of `struct`, as a C compiler lays it out from the header itself."""
    import subprocess
    import tempfile

    inc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include")
    src = "#include <stddef.h>\n#include <stdio.h>\n#include \"%s\"\nint main(void) {\n" % header
    src += '  printf("%%zu\\n", sizeof(%s));\n' % struct
    for f in fields:
        src += '  printf("%s %%zu\\n", offsetof(%s, %s));\n' % (f, struct, f)
    src += "  return 0;\n}\n"
    with tempfile.TemporaryDirectory() as d:
        c, exe = os.path.join(d, "layout.c"), os.path.join(d, "layout")
        with open(c, "w") as fh:
            fh.write(src)
        subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", f"-I{inc}", c, "-o", exe], check=True)
        out = subprocess.run([exe], check=True, capture_output=True, text=True).stdout.split("\n")
    return int(out[0]), {l.split()[0]: int(l.split()[1]) for l in out[1:] if l}


@pytest.mark.parametrize("header,struct,mirror", [("fa_fwd.h", "fa_fwd_params", capi.FaFwdParams),
                                                  ("fa_bwd.h", "fa_bwd_params", capi.FaBwdParams)])
def test_ctypes_mirrors_match_the_headers(header, struct, mirror):
    """The ctypes structures are kept in step with include/*.h by hand: a field added to a header without its mirror (or
    the other way round, or in another order) must fail here, not read past the end of a short struct on the GPU."""
    import re

    names = [f[0] for f in mirror._fields_]
    size, offs = _c_layout(header, struct, names)
    assert ctypes.sizeof(mirror) == size
    for n in names:
        assert getattr(mirror, n).offset == offs[n], n
    # and the header declares no field the mirror lacks
    inc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include", header)
    text = open(inc).read()
    body = text[text.index("typedef struct " + struct):text.index("} " + struct + ";")]
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    declared = []
    for stmt in body.split("{", 1)[1].split(";"):
        stmt = stmt.strip()
        if not stmt:
            continue
        for part in stmt.split(","):
            declared.append(re.findall(r"[A-Za-z_][A-Za-z_0-9]*", part)[-1])
    assert declared == names


def test_host_glue_is_clean_under_asan_and_ubsan():
    """The host-only half of the launchers (validation, kernel choice, workspace sizes for both directions) built with
    the address and undefined-behaviour sanitizers and pushed through ~2.5 million ordinary, extreme (INT32_MAX sizes,
    INT64 strides) and malformed parameter blocks: any overflow or out-of-bounds access aborts the driver."""
    import shutil
    import subprocess
    import tempfile

    if shutil.which("g++") is None:
        pytest.skip("no host C++ compiler")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    with tempfile.TemporaryDirectory() as d:
        exe = os.path.join(d, "host_sanitize")
        subprocess.run(["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-static-libasan", "-fno-sanitize-recover=all", "-Wall",
                        "-Werror", "-I" + os.path.join(root, "include"), "-I" + os.path.join(root, "torch_mlu_amd", "csrc"),
                        os.path.join(root, "tests", "host_sanitize.cpp"), "-o", exe], check=True)
        res = subprocess.run([exe], capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-2000:]
    assert re.match(r"\d+ blocks", res.stdout)


def test_build_refuses_spilling_backward_kernels():
    """The build-time check on compiler output, fed with made-up compiler text: the head_dim-256 backward kernels must
    not use scratch memory, and a build whose remarks do not mention them has not run the check."""
    from torch_mlu_amd import _build

    def remarks(name, scratch):
        return (f"x.hip:130:1: remark: Function Name: {name} [-Rpass-analysis=kernel-resource-usage]\n"
                "  130 | __global__ void k() {\n      | ^\n"
                "x.hip:130:1: remark:     VGPRs: 256 [-Rpass-analysis=kernel-resource-usage]\n"
                f"x.hip:130:1: remark:     ScratchSize [bytes/lane]: {scratch} [-Rpass-analysis=kernel-resource-usage]\n")

    dq256 = "_ZN12_GLOBAL__N_116fa_bwd_dq_kernelIDF16bLi256ELb0ELi0EEEvNS_5BArgsE"
    dkv256 = "_ZN12_GLOBAL__N_117fa_bwd_dkv_kernelIDF16_Li256ELi1ELb0ELb0EEEvNS_5BArgsE"
    dq128 = "_ZN12_GLOBAL__N_116fa_bwd_dq_kernelIDF16bLi128ELb0ELi2EEEvNS_5BArgsE"
    _build.check_bwd256_scratch(remarks(dq256, 0) + remarks(dkv256, 0) + remarks(dq128, 28))   # 128: not this check's business
    with pytest.raises(RuntimeError, match="spills 76 bytes"):
        _build.check_bwd256_scratch(remarks(dq256, 0) + remarks(dkv256, 76))
    with pytest.raises(RuntimeError, match="check not run"):
        _build.check_bwd256_scratch(remarks(dq128, 0))

"""CPU-side checks of the C-ABI boundary: the library loads, exports every
symbol the header declares, and rejects bad arguments on the host before any
launch (so these calls are safe without a GPU)."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "lvx.h")


@pytest.fixture(scope="module")
def lib():
    from lv_xattn import _lib
    if not os.path.exists(_lib.LIB_PATH):
        import importlib.util
        spec = importlib.util.spec_from_file_location("lvx_build", os.path.join(ROOT, "lv-xattn_amd", "build.py"))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        mod.build(force=False)
    return _lib.load()


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lvx_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound(lib):
    from lv_xattn import _lib
    names = declared_symbols()
    assert len(names) >= 10
    for n in names:
        assert hasattr(lib, n), f"{n} declared in lvx.h but not exported by liblvx.so"
    assert sorted(_lib.SYMBOLS) == names, "ctypes table and header disagree"


def test_version_and_error_strings(lib):
    assert lib.lvx_version() == 103
    assert lib.lvx_strerror(0) == b"ok"
    for code in range(-8, 0):
        assert lib.lvx_strerror(code) not in (b"", b"unknown lvx error")


def _shape(**kw):
    from lv_xattn._lib import AttnShape
    d = dict(B=1, Hq=8, Hkv=2, D=128, Lq=64, Lkv=256, dtype=1, scale=0.1, kv_len=None, kv_start=None, kv_end=None)
    d.update(kw)
    return AttnShape(**d)


def _t(ptr=0x1000, sb=8 * 64 * 128, sh=64 * 128, ss=128):
    from lv_xattn._lib import Tensor4
    return Tensor4(ptr, sb, sh, ss)


def _fwd(lib, shape, q=None, k=None, v=None, o=None, lse=0x2000, rb=0, rc=64, splits=1, ws=None, wsb=0):
    q, k, v, o = (x if x is not None else _t() for x in (q, k, v, o))
    return lib.lvx_fwd(C.byref(shape), C.byref(q), C.byref(k), C.byref(v), C.byref(o), lse, rb, rc, splits, ws, wsb, None)


def test_the_build_entry_point_accepts_the_library_it_built(lib):
    # build() of the driver's entry file ends with this check; it reads the version from the header
    import importlib.util
    spec = importlib.util.spec_from_file_location("graft_entry", os.path.join(ROOT, "__graft_entry__.py"))
    entry = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(entry)
    entry.check_abi_version(lib)

    class Stale:
        @staticmethod
        def lvx_version():
            return lib.lvx_version() - 1

    with pytest.raises(RuntimeError, match="ABI"):
        entry.check_abi_version(Stale)


def test_forward_rejects_bad_arguments_before_launch(lib):
    assert _fwd(lib, _shape(D=96)) == -4               # 16, 32, 64 and 128 have kernels
    assert _fwd(lib, _shape(D=256)) == -4
    assert _fwd(lib, _shape(dtype=3)) == -5            # 1 = bf16, 2 = fp16
    assert _fwd(lib, _shape(Hq=7)) == -3
    assert _fwd(lib, _shape(scale=0.0)) == -6
    assert _fwd(lib, _shape(scale=float("nan"))) == -6
    assert _fwd(lib, _shape(), q=_t(ptr=0)) == -1
    assert _fwd(lib, _shape(), k=_t(ptr=0x1004)) == -2
    assert _fwd(lib, _shape(), v=_t(ss=132)) == -2
    assert _fwd(lib, _shape(), lse=None) == -1
    assert _fwd(lib, _shape(), rb=32, rc=64) == -3
    assert _fwd(lib, _shape(), splits=0) == -3
    assert _fwd(lib, _shape(), splits=4) == -7            # no workspace given
    assert _fwd(lib, _shape(kv_start=0x3000)) == -1       # kv_start without kv_end
    assert _fwd(lib, _shape(), rc=0) == 0                 # empty window: nothing to do
    assert lib.lvx_fwd(None, None, None, None, None, None, 0, 0, 1, None, 0, None) == -1


def test_dense_bias_must_be_aligned_for_16_byte_loads(lib):
    ok = dict(bias=0x8000, bias_stride_b=64 * 256, bias_stride_h=0, bias_stride_r=256)
    assert _fwd(lib, _shape(**ok), rc=0) == 0                       # accepted (no rows: nothing is launched)
    assert _fwd(lib, _shape(**dict(ok, bias=0x8004))) == -2         # base not 16-byte aligned
    assert _fwd(lib, _shape(**dict(ok, bias_stride_r=257))) == -2   # rows would start off a 16-byte boundary
    assert _fwd(lib, _shape(**dict(ok, bias_stride_b=64 * 256 + 2))) == -2
    assert _fwd(lib, _shape(**dict(ok, bias_stride_h=6))) == -2
    assert _fwd(lib, _shape(**dict(ok, bias_stride_r=252))) == -3   # shorter than Lkv rounded up to 4


def test_workspace_size(lib):
    s = _shape()
    assert lib.lvx_fwd_workspace_bytes(C.byref(s), 64, 1) == 0
    assert lib.lvx_fwd_workspace_bytes(C.byref(s), 64, 4) == 4 * 8 * 64 * (128 * 2 + 4)


def test_other_entry_points_reject_bad_arguments(lib):
    s = _shape()
    t = _t()
    assert lib.lvx_merge(C.byref(s), C.byref(t), None, C.byref(t), 0x2000, 0, 64, None) == -1
    assert lib.lvx_merge(C.byref(s), C.byref(t), 0x2000, C.byref(t), 0x2000, 0, 65, None) == -3
    assert lib.lvx_bwd_preprocess(C.byref(s), C.byref(t), C.byref(_t(ptr=8)), 0x2000, 0, 64, None) == -2
    assert lib.lvx_bias_hull(C.byref(s), 0x2000, 0x3000, None) == -1          # a shape without a bias
    # lvx_fwd_acc: the accumulator must be there, aligned, and not the output itself
    o_in = _t(ptr=0x9000)
    assert lib.lvx_fwd_acc(C.byref(s), C.byref(t), C.byref(t), C.byref(t), None, 0x2000, C.byref(t), 0x2000,
                           0, 64, 1, None, 0, None) == -1
    assert lib.lvx_fwd_acc(C.byref(s), C.byref(t), C.byref(t), C.byref(t), C.byref(o_in), None, C.byref(t), 0x2000,
                           0, 64, 1, None, 0, None) == -1
    assert lib.lvx_fwd_acc(C.byref(s), C.byref(t), C.byref(t), C.byref(t), C.byref(_t(ptr=8)), 0x2000, C.byref(t),
                           0x2000, 0, 64, 1, None, 0, None) == -2
    assert lib.lvx_fwd_acc(C.byref(s), C.byref(t), C.byref(t), C.byref(t), C.byref(t), 0x2000, C.byref(t), 0x2000,
                           0, 64, 1, None, 0, None) == -3
    # ... nor may the accumulator's LSE be the output's, or the two O windows overlap at another base
    assert lib.lvx_fwd_acc(C.byref(s), C.byref(t), C.byref(t), C.byref(t), C.byref(o_in), 0x2000, C.byref(t), 0x2000,
                           0, 64, 1, None, 0, None) == -3
    assert lib.lvx_fwd_acc(C.byref(s), C.byref(t), C.byref(t), C.byref(t), C.byref(o_in), 0x2100, C.byref(t), 0x2000,
                           0, 64, 1, None, 0, None) == -3
    assert lib.lvx_fwd_acc(C.byref(s), C.byref(t), C.byref(t), C.byref(t), C.byref(_t(ptr=0x1100)), 0x800000,
                           C.byref(t), 0x2000, 0, 64, 1, None, 0, None) == -3
    assert lib.lvx_fwd_acc(C.byref(s), C.byref(t), C.byref(t), C.byref(t), C.byref(o_in), 0x800000, C.byref(t), 0x2000,
                           0, 0, 1, None, 0, None) == 0          # no rows: accepted, nothing launched
    assert lib.lvx_bwd(C.byref(s), C.byref(t), C.byref(t), C.byref(t), C.byref(t), 0x2000, None, C.byref(t),
                       C.byref(t), C.byref(t), 0, 0, 64, 0x4000, 1 << 30, None) == -1
    assert lib.lvx_bwd(C.byref(s), C.byref(t), C.byref(t), C.byref(t), C.byref(t), 0x2000, 0x2000, C.byref(t),
                       C.byref(t), C.byref(t), 2, 0, 64, 0x4000, 1 << 30, None) == -3
    need = lib.lvx_bwd_workspace_bytes(C.byref(s), 64)
    # dS^T tiles + fp32 dK/dV scratch + row metadata records (2 floats per row and head)
    # + fp32 dQ partial tiles (a window this small splits the dQ contraction over the tokens:
    # 2 token blocks, one slice each)
    assert need == 8 * 256 * 64 * 2 + 2 * 256 * 2 * 128 * 4 + 8 * 64 * 2 * 4 + 2 * 8 * 64 * 128 * 4
    # an interval mask adds the live-tile tables: one hull (2 ints, padded to 16 bytes) for the
    # single 256-row group and 8 ints per token block
    sm = _shape(kv_start=0x3000, kv_end=0x3100)
    assert lib.lvx_bwd_workspace_bytes(C.byref(sm), 64) == need + 16 + 2 * 8 * 4 + 16
    assert lib.lvx_bwd(C.byref(s), C.byref(t), C.byref(t), C.byref(t), C.byref(t), 0x2000, 0x2000, C.byref(t),
                       C.byref(t), C.byref(t), 0, 0, 64, 0x4000, need - 1, None) == -7
    assert lib.lvx_bwd(C.byref(s), C.byref(t), C.byref(t), C.byref(t), C.byref(t), 0x2000, 0x2000, C.byref(t),
                       C.byref(t), C.byref(t), 0, 0, 64, None, 0, None) == -7
    # row offsets of q and dO are formed in 32 bits: Lq * row stride must stay below 2^31
    big = _shape(Lq=1 << 20, Lkv=128)
    wide = _t(sb=1 << 40, sh=1 << 33, ss=2048)          # 2^20 rows x 2048 elements = 2^31
    need_big = lib.lvx_bwd_workspace_bytes(C.byref(big), 64)
    assert lib.lvx_bwd(C.byref(big), C.byref(wide), C.byref(t), C.byref(t), C.byref(t), 0x2000, 0x2000, C.byref(t),
                       C.byref(t), C.byref(t), 0, 0, 64, 0x4000, need_big, None) == -8
    assert lib.lvx_bwd(C.byref(big), C.byref(t), C.byref(t), C.byref(t), C.byref(wide), 0x2000, 0x2000, C.byref(t),
                       C.byref(t), C.byref(t), 0, 0, 64, 0x4000, need_big, None) == -8
    assert b"not supported" in lib.lvx_strerror(-8)
    assert lib.lvx_cast_f32(0x1000, C.byref(t), 1, 8, 64, 96, 1, None) == -4
    assert lib.lvx_kv_proj(0x1000, 512, 0x2000, 0x3000, 256, 1, 0x4000, 0x5000, 256, 100, 512, 250, 1, None) == -3
    assert lib.lvx_kv_proj(0x1000, 512, None, 0x3000, 256, 1, 0x4000, 0x5000, 256, 100, 512, 256, 2, None) == -1
    assert lib.lvx_dx_vis(0x1000, 0x1100, 256, 0x2000, 0x3000, 250, 1, 0x4000, 512, 100, 512, 256, 1, None) == -2
    assert lib.lvx_dw_kv(0x1000, 512, 0x1100, 0x1200, 256, 0x2000, 0x3000, 128, 1, 100, 512, 256, 1, None) == -3
    # the second operand pair is optional (single projection) but must be given or omitted as a pair
    assert lib.lvx_kv_proj(0x1000, 512, 0x2000, 0x3000, 256, 1, 0x4000, None, 256, 100, 512, 256, 1, None) == -1
    assert lib.lvx_dx_vis(0x1000, None, 256, 0x2000, 0x3000, 256, 1, 0x4000, 512, 100, 512, 256, 1, None) == -1
    assert lib.lvx_dw_kv(0x1000, 512, 0x1100, 0x1200, 256, 0x2000, None, 256, 1, 100, 512, 256, 1, None) == -1
    # the fused norm needs whole heads of 128 columns and its weight
    assert lib.lvx_kv_proj_norm(0x1000, 512, 0x2000, 0x3000, 192, 1, 0x4000, 0x5000, 192, 100, 512, 192,
                                0x6000, 1e-5, None, None, 1, None) == -4
    assert lib.lvx_kv_proj_norm(0x1000, 512, 0x2000, 0x3000, 256, 1, 0x4000, 0x5000, 256, 100, 512, 256,
                                None, 1e-5, None, None, 1, None) == -1
    assert lib.lvx_k_norm_bwd(0x1000, 256, 0x2000, 256, None, 0x3000, 0x4000, 256, None, 100, 256, 1, None) == -1
    # element types: 1 = bf16, 2 = fp16, anything else is refused
    assert lib.lvx_kv_proj(0x1000, 512, 0x2000, 0x3000, 256, 1, 0x4000, 0x5000, 256, 100, 512, 256, 3, None) == -5
    assert lib.lvx_cast_f32(0x1000, C.byref(t), 1, 8, 64, 128, 0, None) == -5


def test_missing_library_fails_loudly(monkeypatch):
    from lv_xattn import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/liblvx.so")
    with pytest.raises(_lib.LvxError, match="no CPU fallback"):
        _lib.load()


C_CALLER = r"""
#include <dlfcn.h>
#include <stdio.h>
#include <string.h>
#include "lvx.h"

int main(int argc, char** argv) {
    void* h = dlopen(argv[1], RTLD_NOW | RTLD_LOCAL);
    if (!h) { fprintf(stderr, "%s\n", dlerror()); return 2; }
    int (*version)(void) = (int (*)(void))dlsym(h, "lvx_version");
    const char* (*strerr)(int) = (const char* (*)(int))dlsym(h, "lvx_strerror");
    int (*fwd)(const lvx_attn_shape*, const lvx_tensor*, const lvx_tensor*, const lvx_tensor*, const lvx_tensor*,
               float*, int32_t, int32_t, int32_t, void*, size_t, void*) =
        (int (*)(const lvx_attn_shape*, const lvx_tensor*, const lvx_tensor*, const lvx_tensor*, const lvx_tensor*,
                 float*, int32_t, int32_t, int32_t, void*, size_t, void*))dlsym(h, "lvx_fwd");
    size_t (*ws)(const lvx_attn_shape*, int32_t, int32_t) =
        (size_t (*)(const lvx_attn_shape*, int32_t, int32_t))dlsym(h, "lvx_fwd_workspace_bytes");
    if (!version || !strerr || !fwd || !ws) return 3;
    lvx_attn_shape s;
    memset(&s, 0, sizeof s);
    s.B = 1; s.Hq = 8; s.Hkv = 2; s.D = 96; s.Lq = 64; s.Lkv = 256; s.dtype = LVX_BF16; s.scale = 0.125f;
    lvx_tensor t = {(void*)0x1000, 8 * 64 * 128, 64 * 128, 128};
    int rc = fwd(&s, &t, &t, &t, &t, (float*)0x2000, 0, 64, 1, NULL, 0, NULL);   /* rejected on the host: D is none of 16, 32, 64, 128 */
    s.D = 128;
    printf("%d|%d|%s|%zu\n", version(), rc, strerr(rc), ws(&s, 64, 4));
    return 0;
}
"""


def test_plain_c_caller_compiles_against_the_header_and_calls_the_library(lib, tmp_path):
    """The boundary is a C ABI: a C99 translation unit including lvx.h builds with gcc, loads
    the library and gets the host-side argument check (no GPU involved)."""
    import shutil
    import subprocess
    from lv_xattn import _lib
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    src = tmp_path / "caller.c"
    src.write_text(C_CALLER)
    exe = tmp_path / "caller"
    subprocess.run([gcc, "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe), "-ldl"],
                   check=True, capture_output=True, text=True)
    r = subprocess.run([str(exe), _lib.LIB_PATH], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    version, rc, msg, ws = r.stdout.strip().split("|")
    assert int(version) == 103 and int(rc) == -4 and msg == "head_dim must be 16, 32, 64 or 128"
    assert int(ws) == 4 * 8 * 64 * (128 * 2 + 4)

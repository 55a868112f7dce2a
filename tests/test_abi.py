"""The C-ABI library loads without a GPU and exports exactly what include/monarch_hip.h declares."""
import ctypes as C
import os
import re
import subprocess

from monarch_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "monarch_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return set(re.findall(r"\b(mhip_[a-z0-9_]+)\s*\(", text))


def test_header_binding_and_library_agree():
    decl = declared_symbols()
    assert decl == set(_lib.SIGNATURES), decl ^ set(_lib.SIGNATURES)
    lib = _lib.lib()  # binds every symbol or raises
    for name in decl:
        assert hasattr(lib, name)
    out = subprocess.run(["nm", "-D", "--defined-only", _lib.LIB_PATH], capture_output=True, text=True).stdout
    exported = set(re.findall(r"\bT (mhip_[a-z0-9_]+)", out))
    assert decl <= exported, decl - exported


def test_header_compiles_as_plain_c():
    src = '#include "monarch_hip.h"\nint main(void) { mhip_slice_t s; (void)s; return MHIP_SUCCESS; }\n'
    r = subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), "-x", "c", "-",
                        "-fsyntax-only"], input=src, text=True, capture_output=True)
    assert r.returncode == 0, r.stderr


def test_status_text_and_host_only_calls():
    lib = _lib.lib()
    assert lib.mhip_version() >= 100
    assert b"stride" in lib.mhip_error_string(_lib.ERR_STRIDE_TOO_SMALL)
    assert b"float8" in lib.mhip_error_string(_lib.ERR_FLOAT8_REDUCTION)
    assert lib.mhip_error_string(0) == b"success"
    assert lib.mhip_dtype_size(_lib.DTYPE_BF16) == 2 and lib.mhip_dtype_size(_lib.DTYPE_F64) == 8
    assert lib.mhip_dtype_size(2) == 0
    # argument checks that precede any launch run without a GPU (torch-sys-cuda/src/nccl.rs:300-316,474-476)
    one = (C.c_void_p * 1)(16)
    assert lib.mhip_reduce(16, one, 1, 4, _lib.DTYPE_F8E4M3FN, 0, None) == _lib.ERR_FLOAT8_REDUCTION
    assert lib.mhip_reduce(16, one, 1, 4, 2, 0, None) == _lib.ERR_INVALID_DATA_TYPE
    assert lib.mhip_reduce(16, one, 1, 4, _lib.DTYPE_F32, 5, None) == _lib.ERR_UNSUPPORTED_OP
    assert lib.mhip_reduce(16, one, 1, 4, _lib.DTYPE_F32, -1, None) == _lib.ERR_UNSUPPORTED_OP
    assert lib.mhip_reduce(16, one, 1, 4, _lib.DTYPE_I32, 4, None) == _lib.ERR_UNSUPPORTED_OP
    assert lib.mhip_reduce(16, one, 0, 4, _lib.DTYPE_F32, 0, None) == _lib.ERR_INVALID_ARGUMENT
    many = (C.c_void_p * 65)(*([16] * 65))
    assert lib.mhip_reduce(16, many, 65, 4, _lib.DTYPE_F32, 0, None) == _lib.ERR_TOO_MANY_INPUTS
    assert lib.mhip_reduce(None, one, 1, 4, _lib.DTYPE_F32, 0, None) == _lib.ERR_UNDEFINED_TENSOR
    assert lib.mhip_reduce(16, one, 1, 0, _lib.DTYPE_F32, 0, None) == 0  # nothing to do
    assert lib.mhip_fp8_quantize(16, 16, 16, 10, 512, None) == _lib.ERR_UNSUPPORTED_BLOCK
    from monarch_amd import Slice
    bad = Slice(offset=0, sizes=[2, 2], strides=[2, 2], _validate=False)
    assert lib.mhip_slice_pack(16, 16, C.byref(bad.c), 4, None) == _lib.ERR_NONUNIQUE_STRIDES
    empty = Slice(offset=0, sizes=[0], strides=[1])
    assert lib.mhip_slice_pack(None, None, C.byref(empty.c), 4, None) == 0
    # staging slots are never a multiple of 16 KiB apart, and always at least a slot apart
    pitch = C.c_size_t()
    for nbytes in (1, 8191, 8192, 16384, 16385, 50331648, 33554432, 3 * 16384 + 8192):
        assert lib.mhip_staging_slot_pitch(nbytes, C.byref(pitch)) == 0
        assert pitch.value >= nbytes and pitch.value % 16384 == 8192 and pitch.value - nbytes < 16384 + 8192
    assert lib.mhip_staging_slot_pitch(0, C.byref(pitch)) == _lib.ERR_INVALID_ARGUMENT
    assert lib.mhip_staging_slot_pitch(2**64 - 1, C.byref(pitch)) == _lib.ERR_INVALID_ARGUMENT


def test_fastdiv_exhaustive_on_host(tmp_path):
    src = r'''
#include "fastdiv.h"
#include <cstdio>
#include <cstdint>
int main() {
  const uint32_t ds[] = {1,2,3,5,7,8,9,10,224,255,256,257,1000,1792,4096,14336,65535,65536,65537,1000003,
                         0x3fffffffu,0x40000000u,0x40000001u,0x7ffffffdu,0x7ffffffeu};
  uint64_t bad = 0;
  for (uint32_t d : ds) {
    mhip::FastDiv32 f(d);
    for (uint64_t n = 0; n < 0x7fffffffull; n += (n < 70000 ? 1 : 9973)) {
      uint32_t q, r; f.divmod((uint32_t)n, q, r);
      if (q != n / d || r != n % d) ++bad;
    }
    for (uint64_t n = 0x7fffffffull - 70000; n < 0x7fffffffull; ++n) {
      if (f.div((uint32_t)n) != n / d) ++bad;
    }
    for (uint64_t k = 1; k * d < 0x7fffffffull && k < 200000; ++k) {  // multiples and their neighbours
      uint64_t n = k * d;
      if (f.div((uint32_t)n) != k || f.div((uint32_t)(n - 1)) != (n - 1) / d) ++bad;
    }
  }
  std::printf("%llu\n", (unsigned long long)bad);
  return bad != 0;
}
'''
    cpp = tmp_path / "t.cpp"
    cpp.write_text(src)
    exe = tmp_path / "t"
    subprocess.check_call(["g++", "-O2", "-std=c++17", "-I", os.path.join(ROOT, "monarch_amd", "csrc"), str(cpp), "-o", str(exe)])
    r = subprocess.run([str(exe)], capture_output=True, text=True)
    assert r.returncode == 0 and r.stdout.strip() == "0", r.stdout


def test_rust_extern_block_names_match_header():
    text = open(os.path.join(ROOT, "hip-sys", "src", "lib.rs")).read()
    rust = set(re.findall(r"pub fn (mhip_[a-z0-9_]+)\(", text))
    assert rust == declared_symbols(), rust ^ declared_symbols()
    # status codes in the Rust module equal the header's
    header = open(os.path.join(ROOT, "include", "monarch_hip.h")).read()
    for name, value in re.findall(r"MHIP_ERR_([A-Z0-9_]+) = (\d+)", header):
        assert re.search(rf"pub const {name}: i32 = {value};", text), name


# C parameter / return types of the header -> the Rust spelling the extern block must use
_RUST_TYPE = {
    "const float*": "*const f32", "const float* const*": "*const *const f32", "const mhip_slice_t*": "*const mhip_slice_t",
    "const uint32_t*": "*const u32", "const uint64_t*": "*const u64", "const uint8_t*": "*const u8",
    "const uint8_t* const*": "*const *const u8", "const void*": "*const c_void", "const void* const*": "*const *const c_void",
    "float*": "*mut f32", "int": "c_int", "int*": "*mut c_int", "mhip_event_t": "mhip_event_t",
    "mhip_event_t*": "*mut mhip_event_t", "mhip_stream_t": "mhip_stream_t", "mhip_stream_t*": "*mut mhip_stream_t",
    "size_t": "usize", "size_t*": "*mut usize", "uint32_t": "u32", "uint64_t": "u64", "uint64_t*": "*mut u64",
    "uint8_t*": "*mut u8", "void*": "*mut c_void", "void* const*": "*const *mut c_void", "void**": "*mut *mut c_void",
    "const char*": "*const c_char", "const char* const*": "*const *const c_char", "uint32_t*": "*mut u32",
    "const mhip_rdma_buffer_t*": "*const mhip_rdma_buffer_t", "const size_t*": "*const usize",
    "const mhip_wqe_params_t*": "*const mhip_wqe_params_t", "const mhip_cqe_poll_params_t*": "*const mhip_cqe_poll_params_t",
    "int32_t*": "*mut i32",
}


def test_rust_extern_block_types_match_header():
    # every parameter and return type of the Rust declarations is the header's, spelled in Rust: no `*mut` for a
    # `const` pointer, no `usize` for a `uint64_t`, out-parameters as `*mut`
    header = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "monarch_hip.h")).read(), flags=re.S)
    rust = open(os.path.join(ROOT, "hip-sys", "src", "lib.rs")).read()
    rust_decl = {name: (params, ret) for name, params, ret in
                 re.findall(r"pub fn (mhip_[a-z0-9_]+)\(([^()]*)\) -> ([^;]+);", rust)}
    protos = re.findall(r"^\s*([A-Za-z_][A-Za-z0-9_ \*]*?)\s*\b(mhip_[a-z0-9_]+)\s*\(([^()]*)\)\s*;", header, flags=re.M)
    assert len(protos) == len(declared_symbols())
    for ret, name, params in protos:
        want = []
        for p in params.split(","):
            p = " ".join(p.split())
            if p in ("", "void"):
                continue
            ctype = re.match(r"(.*?)([A-Za-z_][A-Za-z0-9_]*)$", p).group(1).strip().replace(" *", "*")
            want.append(_RUST_TYPE[ctype])
        got_params, got_ret = rust_decl[name]
        got = [a.split(":", 1)[1].strip() for a in got_params.split(",") if a.strip()]
        assert got == want, (name, got, want)
        assert got_ret.strip() == _RUST_TYPE[" ".join(ret.split()).replace(" *", "*")], (name, got_ret)


def test_ctypes_table_scalar_widths_match_header():
    # scalars are passed by value: a wrong width in the ctypes table shifts every later argument.  Pointers may be
    # declared as c_void_p or as a typed POINTER in the table; both are pointer-sized.
    import ctypes as C
    scalar = {"int": C.c_int, "uint32_t": C.c_uint32, "uint64_t": C.c_uint64, "size_t": C.c_size_t}
    header = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "monarch_hip.h")).read(), flags=re.S)
    protos = re.findall(r"^\s*([A-Za-z_][A-Za-z0-9_ \*]*?)\s*\b(mhip_[a-z0-9_]+)\s*\(([^()]*)\)\s*;", header, flags=re.M)
    for ret, name, params in protos:
        restype, argtypes = _lib.SIGNATURES[name]
        ctypes_of = []
        for p in params.split(","):
            p = " ".join(p.split())
            if p in ("", "void"):
                continue
            ctypes_of.append(re.match(r"(.*?)([A-Za-z_][A-Za-z0-9_]*)$", p).group(1).strip().replace(" *", "*"))
        for i, (ct, at) in enumerate(zip(ctypes_of, argtypes)):
            if ct in scalar:
                assert C.sizeof(at) == C.sizeof(scalar[ct]) and not hasattr(at, "contents") and at is not C.c_void_p, (name, i, ct, at)
            else:  # every other parameter type of the header is a pointer or an opaque handle
                assert C.sizeof(at) == C.sizeof(C.c_void_p), (name, i, ct, at)
        ret = " ".join(ret.split()).replace(" *", "*")
        assert C.sizeof(restype) == (C.sizeof(scalar[ret]) if ret in scalar else C.sizeof(C.c_void_p)), (name, ret)


def _param_counts(text, pattern):
    counts = {}
    for name, params in re.findall(pattern, text, flags=re.S):
        params = params.strip()
        counts[name] = 0 if params in ("", "void") else params.count(",") + 1
    return counts


def test_every_binding_has_the_header_parameter_count():
    # the header, the ctypes table and the Rust extern block declare the same number of parameters per symbol
    header = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "monarch_hip.h")).read(), flags=re.S)
    c_counts = _param_counts(header, r"\b(mhip_[a-z0-9_]+)\s*\(([^()]*)\)\s*;")
    rust = open(os.path.join(ROOT, "hip-sys", "src", "lib.rs")).read()
    rust_counts = _param_counts(rust, r"pub fn (mhip_[a-z0-9_]+)\(([^()]*)\)")
    assert set(c_counts) == set(_lib.SIGNATURES) == set(rust_counts)
    for name, n in c_counts.items():
        assert len(_lib.SIGNATURES[name][1]) == n, (name, "ctypes", len(_lib.SIGNATURES[name][1]), n)
        assert rust_counts[name] == n, (name, "rust", rust_counts[name], n)


def test_product_never_touches_the_oracle_and_fails_loudly_without_the_library(monkeypatch, tmp_path):
    import monarch_amd
    pkg = os.path.dirname(monarch_amd.__file__)
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".cpp", ".h")) or f == "Makefile":
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower(), os.path.join(dirpath, f)
    # no CPU fallback: a missing shared library is an error at the first call
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libmonarch_hip.so"))
    import pytest
    with pytest.raises(_lib.MonarchHipNotBuilt):
        monarch_amd.Slice(offset=0, sizes=[2], strides=[1])


def test_overflowing_slices_are_refused_on_the_host():
    from monarch_amd import Slice
    lib = _lib.lib()
    big = 1 << 62
    assert lib.mhip_slice_validate(0, _lib.u64_array([8, 2]), 2, _lib.u64_array([big, 1]), 2) == _lib.ERR_INVALID_ARGUMENT
    s = Slice(offset=1 << 62, sizes=[4], strides=[1])           # valid as a Slice, not addressable at 8 bytes/element
    assert lib.mhip_slice_pack(16, 16, C.byref(s.c), 8, None) == _lib.ERR_INVALID_ARGUMENT
    t = Slice(offset=0, sizes=[1 << 40, 1 << 30], strides=[1 << 30, 1], _validate=False)
    assert lib.mhip_slice_pack(16, 16, C.byref(t.c), 1, None) == _lib.ERR_INVALID_ARGUMENT


def test_the_library_reads_the_environment_only_while_it_loads():
    # entry points may be called from any thread while the host application changes its environment, and a stray
    # variable must not change kernel selection: the only getenv calls are the two load-time initialisers of runtime.cpp
    # and tuning_env(), which asks only when MONARCH_HIP_TUNING=1 was set at load time
    src = os.path.join(ROOT, "monarch_amd", "csrc")
    uses = []
    for f in sorted(os.listdir(src)):
        if f.endswith((".hip", ".cpp", ".h")):
            text = re.sub(r"//[^\n]*", "", open(os.path.join(src, f)).read())
            uses += [(f, m.start()) for m in re.finditer(r"\bgetenv\s*\(", text)]
    files = [f for f, _ in uses]
    assert files.count("runtime.cpp") == 3 and files.count("mhip_device.h") == 1 and len(files) == 4, uses
    device_h = open(os.path.join(src, "mhip_device.h")).read()
    assert "return g_tuning ? std::getenv(name) : nullptr;" in device_h
    runtime = open(os.path.join(src, "runtime.cpp")).read()
    first_fn = runtime.index('extern "C"')
    assert all(m.start() < first_fn for m in re.finditer(r"\bgetenv\s*\(", runtime))   # namespace-scope initialisers only


def test_packed_fp32_instructions_are_off_in_device_code(tmp_path):
    # the build switches v_pk_{add,mul,fma}_f32 off; the x86 host pass does not know the AMDGPU feature and says so,
    # the device pass honours it: a float2 multiply-add compiled with the Makefile's flags holds none of them
    flags = subprocess.run(["make", "-s", "-C", os.path.join(ROOT, "monarch_amd", "csrc"), "print-hipflags"], capture_output=True,
                           text=True).stdout.split()
    assert "-packed-fp32-ops" in flags
    src = tmp_path / "k.hip"
    src.write_text("#include <hip/hip_runtime.h>\n__global__ void k(float2* a, const float2* b, const float2* c) {\n"
                   "  int i = blockIdx.x * blockDim.x + threadIdx.x; float2 x = b[i], y = c[i], z = a[i];\n"
                   "  z.x = x.x * y.x + z.x; z.y = x.y * y.y + z.y; z.x += x.x; z.y += x.y; a[i] = z; }\n")

    def packed_ops(extra):
        r = subprocess.run(["/opt/rocm/bin/hipcc", "--offload-arch=gfx950", "-O3", *extra, "-S", "--cuda-device-only", str(src), "-o", "-"],
                           capture_output=True, text=True)
        assert r.returncode == 0, r.stderr
        return len(re.findall(r"\bv_pk_(?:add|mul|fma)_f32\b", r.stdout))

    assert packed_ops([f for f in flags if f not in ("-c",) and not f.startswith("--offload-arch")]) == 0
    assert packed_ops([]) > 0      # the check can fail: without the flag the same source does use them

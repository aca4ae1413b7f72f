"""Loader and builder of libwmmae_tcec.so (the C-ABI declared in include/wmmae_tcec.h).

The library is built in-tree with hipcc for gfx950 and loaded with ctypes.
There is no fallback: if the shared object is missing, `lib()` raises.
"""
import ctypes
import glob
import os
import subprocess

_PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(_PKG)
INCLUDE_DIR = os.path.join(ROOT, "include")
CSRC_DIR = os.path.join(_PKG, "csrc")
LIB_DIR = os.path.join(_PKG, "lib")
# WMMAE_TCEC_LIB names another build of the same library (for comparing two
# builds on one GPU); the default is the in-tree one
LIB_PATH = os.environ.get("WMMAE_TCEC_LIB") or os.path.join(LIB_DIR, "libwmmae_tcec.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # keep the compiler from forming packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]

# every symbol include/wmmae_tcec.h declares
EXPORTS = [
    "wmmae_status_string",
    "wmmae_query",
    "wmmae_tcec_sgemm_workspace_bytes",
    "wmmae_tcec_sgemm_path",
    "wmmae_tcec_sgemm",
    "wmmae_tcec_sgemm_static",
    "wmmae_tcec_sgemm_strided_batched",
    "wmmae_tcec_sgemm_batched",
    "wmmae_tcec_pack_bytes",
    "wmmae_tcec_pack",
    "wmmae_tcec_gemm_packed_workspace_bytes",
    "wmmae_tcec_gemm_packed",
    "wmmae_primitive_tiles",
    "wmmae_layout_dump",
    "wmmae_tcec_mma_tile",
    "wmmae_tcec_mma_tile_native",
    "wmmae_tcec_matvec",
    "wmmae_tcec_frag_dump",
    "wmmae_tcec_elementwise",
    "wmmae_tcec_api_gemm",
    "wmmae_tcec_api_gemm_rounding",
    "wmmae_tcec_api_gemm_batched",
    "wmmae_tcec_mma_complex",
    "wmmae_primitive_mma",
    "wmmae_foreach_ec",
    "wmmae_gevm",
    "wmmae_fragment_ops",
    "wmmae_fragment_eye",
    "wmmae_direct_product",
    "wmmae_clock_samples",
    "wmmae_utils_cp_async",
    "wmmae_utils_cp_async_pipeline",
    "wmmae_print_fragment",
    "wmmae_utils_cast",
    "wmmae_mfma_probe",
    "wmmae_direct_read_first",
    "wmmae_tcec_sgemm_k_slices",
    "wmmae_tcec_force_k_slices",
    "wmmae_tcec_time_gemm_kernel",
    "wmmae_tcec_path_estimates",
    "wmmae_mfma_source_hazard_probe",
]


# one object per translation unit; compiled side by side, then linked
SOURCES = ["capi_gemm.hip", "capi_harness.hip", "capi_api_gemm.hip"]
ASM_MFMA_SOURCES = ["capi_gemm.hip"]


def device_asm_path(name):
    """Where build() leaves the gfx950 assembly of a translation unit with inline-asm MFMAs."""
    return os.path.join(LIB_DIR, name.replace(".hip", "") + "-hip-amdgcn-amd-amdhsa-gfx950.s")


def _run(cmd, verbose):
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if verbose or res.returncode != 0:
        print(res.stdout)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed building libwmmae_tcec.so:\n" + res.stdout[-4000:])


def build(verbose=False, only=None):
    """Compile the HIP sources into LIB_PATH.  Always recompiles every source
    (`only` = list of source names restricts that to a few, the other objects
    being reused if present: for work on one kernel)."""
    from concurrent.futures import ThreadPoolExecutor
    os.makedirs(LIB_DIR, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    flags = [f for f in HIPCC_FLAGS if f != "-shared"]
    objs, jobs = [], []
    for name in SOURCES:
        obj = os.path.join(LIB_DIR, name.replace(".hip", ".o"))
        objs.append(obj)
        if only is None or name in only or not os.path.exists(obj):
            # (the translation units whose kernels issue MFMAs from inline asm keep their
            # device assembly, for the check below)
            keep = ["-save-temps=obj"] if name in ASM_MFMA_SOURCES else []
            jobs.append([hipcc, *flags, *keep, "-I" + INCLUDE_DIR, "-c",
                         os.path.join(CSRC_DIR, name), "-o", obj])
    with ThreadPoolExecutor(max_workers=len(SOURCES)) as pool:
        list(pool.map(lambda c: _run(c, verbose), jobs))
    from . import isa_check
    for name in ASM_MFMA_SOURCES:
        stem = os.path.join(LIB_DIR, name.replace(".hip", ""))
        for f in glob.glob(stem + "-*") + glob.glob(stem + ".hip-*"):
            if not f.endswith("-gfx950.s"):
                os.remove(f)
        # pipeline hazards around the hand-placed MFMAs, which the compiler does not see:
        # no library is linked from code that has one
        isa_check.check_file(device_asm_path(name))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB_PATH], verbose)
    return LIB_PATH


_LIB = None

_c = ctypes
_vp, _i, _ll, _sz = _c.c_void_p, _c.c_int, _c.c_longlong, _c.c_size_t
_fp = _c.POINTER(_c.c_float)

_SIGNATURES = {
    "wmmae_status_string": (_c.c_char_p, [_i]),
    "wmmae_query": (_i, [_i, _c.POINTER(_ll)]),
    "wmmae_tcec_sgemm_workspace_bytes": (_i, [_i, _i, _i, _i, _i, _c.POINTER(_sz)]),
    "wmmae_tcec_sgemm_path": (_i, [_i, _i, _i, _i, _i, _i, _c.POINTER(_i)]),
    "wmmae_tcec_sgemm": (_i, [_c.c_char, _c.c_char, _i, _i, _i, _fp, _vp, _i, _vp, _i, _fp,
                              _vp, _i, _i, _i, _vp, _sz, _vp]),
    "wmmae_tcec_sgemm_static": (_i, [_c.c_char, _c.c_char, _i, _i, _i, _fp, _vp, _i, _vp, _i, _fp,
                                     _vp, _i, _i, _i, _vp]),
    "wmmae_tcec_sgemm_strided_batched": (_i, [_c.c_char, _c.c_char, _i, _i, _i, _fp, _vp, _i, _ll,
                                              _vp, _i, _ll, _fp, _vp, _i, _ll, _i, _i, _i,
                                              _vp, _sz, _vp]),
    "wmmae_tcec_sgemm_batched": (_i, [_c.c_char, _c.c_char, _i, _i, _i, _fp, _vp, _i, _vp, _i, _fp,
                                      _vp, _i, _i, _i, _i, _vp, _sz, _vp]),
    "wmmae_tcec_pack_bytes": (_i, [_i, _i, _i, _i, _c.POINTER(_sz)]),
    "wmmae_tcec_pack": (_i, [_i, _i, _i, _vp, _ll, _ll, _ll, _i, _vp, _sz, _vp]),
    "wmmae_tcec_gemm_packed_workspace_bytes": (_i, [_i, _i, _i, _i, _i, _c.POINTER(_sz)]),
    "wmmae_tcec_gemm_packed": (_i, [_i, _i, _i, _i, _fp, _vp, _vp, _fp, _vp, _i, _ll, _i, _i, _vp, _sz,
                                    _vp]),
    "wmmae_primitive_tiles": (_i, [_vp, _ll, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "wmmae_layout_dump": (_i, [_i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp]),
    "wmmae_tcec_mma_tile": (_i, [_i, _i, _i, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "wmmae_tcec_mma_tile_native": (_i, [_i, _i, _i, _i, _vp, _vp, _vp, _i, _vp]),
    "wmmae_tcec_matvec": (_i, [_i, _i, _vp, _vp, _vp, _i, _i, _vp]),
    "wmmae_tcec_frag_dump": (_i, [_i, _i, _i, _i, _vp, _vp, _i, _i, _vp]),
    "wmmae_tcec_elementwise": (_i, [_i, _i, _i, _vp, _c.c_float, _i, _i, _vp]),
    "wmmae_tcec_api_gemm": (_i, [_i, _i, _i, _i, _i, _fp, _vp, _i, _vp, _i, _fp, _vp, _i, _vp]),
    "wmmae_tcec_api_gemm_rounding": (_i, [_i, _i, _i, _i, _i, _i, _fp, _vp, _i, _vp, _i, _fp, _vp, _i, _vp]),
    "wmmae_tcec_api_gemm_batched": (_i, [_i, _i, _i, _i, _i, _fp, _vp, _i, _vp, _i, _fp, _vp, _i, _i, _vp]),
    "wmmae_tcec_mma_complex": (_i, [_i, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _c.c_float, _vp]),
    "wmmae_primitive_mma": (_i, [_i, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "wmmae_foreach_ec": (_i, [_vp, _vp, _vp, _vp]),
    "wmmae_gevm": (_i, [_vp, _vp, _vp, _vp]),
    "wmmae_fragment_ops": (_i, [_i, _i, _i, _c.c_float, _vp, _vp, _vp, _vp]),
    "wmmae_fragment_eye": (_i, [_i, _i, _c.c_float, _vp, _vp]),
    "wmmae_direct_product": (_i, [_i, _i, _i, _vp, _vp, _vp, _vp]),
    "wmmae_clock_samples": (_i, [_vp, _i, _ll, _vp]),
    "wmmae_utils_cp_async": (_i, [_i, _i, _vp, _vp, _vp]),
    "wmmae_utils_cp_async_pipeline": (_i, [_i, _i, _i, _vp, _vp, _vp, _vp]),
    "wmmae_print_fragment": (_i, [_i, _i, _vp, _c.c_float, _vp]),
    "wmmae_utils_cast": (_i, [_i, _vp, _vp, _ll, _vp]),
    "wmmae_mfma_probe": (_i, [_i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp]),
    "wmmae_direct_read_first": (_i, [_i, _i, _i, _i, _c.POINTER(_ll)]),
    "wmmae_tcec_sgemm_k_slices": (_i, [_i, _i, _i, _i, _i, _i, _c.POINTER(_i)]),
    "wmmae_tcec_force_k_slices": (_i, [_i]),
    "wmmae_tcec_time_gemm_kernel": (_i, [_vp, _vp]),
    "wmmae_tcec_path_estimates": (_i, [_i, _i, _i, _i, _i, _c.POINTER(_c.c_double)]),
    "wmmae_mfma_source_hazard_probe": (_i, [_i, _i, _vp, _vp]),
}


def lib():
    """Return the loaded C-ABI library; raise if it has not been built."""
    global _LIB
    if _LIB is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with __graft_entry__.build() "
                "(hipcc --offload-arch=gfx950); there is no CPU fallback")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in _SIGNATURES.items():
            if not hasattr(handle, name) and os.environ.get("WMMAE_TCEC_LIB"):
                continue          # an older build named for a comparison: fewer entry points
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _LIB = handle
    return _LIB


class WmmaeError(RuntimeError):
    def __init__(self, status, where):
        self.status = status
        msg = lib().wmmae_status_string(status).decode()
        super().__init__(f"{where}: {msg} (status {status})")


def check(status, where):
    if status != 0:
        raise WmmaeError(status, where)

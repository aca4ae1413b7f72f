"""Every include path of the reference's public and detail headers that belongs to this path
exists here under the same name and compiles on its own for gfx950, and the names code reaches
for in `tcec::detail` are there (reference: include/wmma_extension/tcec/tcec.hpp:3-8, 934-936,
tcec/detail/common.hpp:12-82, utils.hpp:29-64).  Compile-only: no GPU is touched."""
import os
import subprocess
import tempfile
from concurrent.futures import ThreadPoolExecutor

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INCLUDE = os.path.join(ROOT, "include")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# the reference's headers for this path (its per-architecture NVIDIA tables sm_*.hpp and
# m16n8k*.hpp have no counterpart: one layout model serves gfx950)
HEADERS = [
    "wmma_extension/wmma_extension.hpp",
    "wmma_extension/wmma_mma.hpp",
    "wmma_extension/operators.hpp",
    "wmma_extension/utils.hpp",
    "wmma_extension/detail/common.hpp",
    "wmma_extension/detail/operators.hpp",
    "wmma_extension/tcec/tcec.hpp",
    "wmma_extension/tcec/complex.hpp",
    "wmma_extension/tcec/detail/common.hpp",
    "wmma_extension/tcec/detail/functions.hpp",
    "wmma_extension/tcec/detail/functions_simt.hpp",
    "wmma_extension/tcec/detail/policy.hpp",
    "wmma_extension/tcec/detail/policy_simt.hpp",
    "wmma_extension/tcec/detail/scale.hpp",
    "wmma_extension/tcec/detail/no_cor.hpp",
    "wmma_extension/tcec/detail/notc.hpp",
    "wmma_extension/tcec/detail/print.hpp",
    "wmma_extension/tcec/detail/wmma_extension_include.hpp",
    "wmma_extension/tcec/detail/wmma_extension_simt_include.hpp",
    "wmma_extension/tcec/detail/simt/mma_simt.hpp",
    "wmma_extension/tcec/detail/simt/detail/common.hpp",
    "wmma_extension/tcec/detail/simt/detail/fma.hpp",
    "wmma_extension/tcec/detail/simt/detail/m16n16k16.hpp",
]

# the fragment namespace behind the reference's op_simt policy, used directly
# (reference: tcec/detail/simt/mma_simt.hpp:9-262, simt/detail/fma.hpp:10-24)
MMA_SIMT = r"""
#include <hip/hip_runtime.h>
#include <wmma_extension/tcec/detail/wmma_extension_simt_include.hpp>
#include <type_traits>
namespace w = mtk::wmma;
namespace s = mtk::wmma::mma_simt;
using frag_a = s::fragment<w::matrix_a, 16, 16, 16, float, w::row_major>;
using frag_b = s::fragment<w::matrix_b, 16, 16, 16, float, w::col_major>;
using frag_c = s::fragment<w::accumulator, 16, 16, 16, float>;
static_assert(std::is_same<frag_a, w::fragment<w::matrix_a, 16, 16, 16, float, w::row_major>>::value, "");
__global__ void k(float *d, const float *a, const float *b, const float *c, float *v) {
  frag_a fa;
  frag_b fb;
  frag_c fc, fd;
  s::load_matrix_sync(fa, a, 16);
  s::load_matrix_sync(fb, b, 16);
  s::load_matrix_sync(fc, c, 16, w::mem_col_major);
  s::mma_sync(fd, fa, fb, fc);
  s::foreach_ij<frag_c>(w::mem_col_major, [&](const unsigned *list, const unsigned n, const unsigned i,
                                              const unsigned j) {
    for (unsigned x = 0; x < n; x++)
      fd.x[list[x]] += s::detail::fma<float, float, float>{}(float(i), float(j), 1.f);
  });
  s::store_matrix_sync(d, fd, 16, w::mem_col_major);
  s::fill_zero(fa);
  s::load_vector(fa, v);
  s::store_vector(v, fd, w::mem_col_major);
  v[20] = float(s::detail::fma<double, double, double>{}(1.0, 2.0, 3.0));
}
"""

DETAIL_NAMES = r"""
#include <hip/hip_runtime.h>
#include <wmma_extension/tcec/detail/common.hpp>
#include <wmma_extension/tcec/detail/scale.hpp>
#include <wmma_extension/tcec/tcec.hpp>
#include <wmma_extension/utils.hpp>
#include <type_traits>
namespace w = mtk::wmma;
namespace d = mtk::wmma::tcec::detail;
static_assert(std::is_same<d::sub_frag_t<w::matrix_a, w::half>::type, w::half>::value, "");
static_assert(std::is_same<d::sub_frag_t<w::matrix_b, w::bfloat16>::type, w::bfloat16>::value, "");
static_assert(std::is_same<d::sub_frag_t<w::accumulator, w::half>::type, float>::value, "");
static_assert(std::is_same<d::sub_frag_t<w::accumulator, w::precision::tf32>::type, float>::value, "");
static_assert(d::get_fragment_k<w::half>() == 32 && d::get_fragment_k<w::precision::tf32>() == 32, "");
static_assert(d::get_fragment_k<float>() == 16, "");
static_assert(d::select_value<w::matrix_a, 1, 2, 3>::value == 1 &&
              d::select_value<w::matrix_b, 1, 2, 3>::value == 2 &&
              d::select_value<w::accumulator, 1, 2, 3>::value == 3, "");
static_assert(d::layout_switch<w::col_major, 5, 7>::value == 5 &&
              d::layout_switch<w::row_major, 5, 7>::value == 7, "");
// the fragment's own sub-fragment element follows sub_frag_t
using frag_a = w::tcec::fragment<w::matrix_a, 32, 32, 32, w::half, w::row_major>;
using frag_c = w::tcec::fragment<w::accumulator, 32, 32, 32, w::half>;
static_assert(std::is_same<frag_a::sub_elem_t, w::half>::value, "");
static_assert(std::is_same<frag_c::sub_elem_t, float>::value, "");
static_assert(frag_a::sub_frag_k == d::get_fragment_k<w::half>(), "");
__global__ void k(float *out, const float *in) {
  __shared__ float tile[3][64];
  namespace cpa = w::utils::cp_async;
  out[0] = static_cast<float>(d::compute_mem_offset<16, 16, w::col_major>{}(3u, 2u, 40u, 16u, 32u)) +
           static_cast<float>(d::compute_mem_offset<16, 16, w::row_major>{}(35u, 40u, 16u, 32u)) +
           d::correction_scale_0<w::half>(1.f) + d::correction_scale_1<w::half>(1.f);
  for (int s = 0; s < 3; s++) {
    cpa::cp_async<4>(&tile[s][threadIdx.x], in + 64 * s + threadIdx.x);
    cpa::commit();
  }
  cpa::wait_group<2>();
  out[1 + threadIdx.x] = tile[0][threadIdx.x];
  cpa::wait_group<1>();
  out[65 + threadIdx.x] = tile[1][threadIdx.x];
  cpa::wait_all();
  out[129 + threadIdx.x] = tile[2][threadIdx.x];
}
"""


def _syntax_only(source):
    with tempfile.TemporaryDirectory() as tmp:
        path = os.path.join(tmp, "t.hip")
        with open(path, "w") as f:
            f.write(source)
        res = subprocess.run(
            [HIPCC, "--offload-arch=gfx950", "-std=c++17", "-fsyntax-only", "-I" + INCLUDE, path],
            stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    return res.returncode, res.stdout


def test_every_reference_include_path_compiles_alone():
    for h in HEADERS:
        assert os.path.exists(os.path.join(INCLUDE, h)), h
    sources = [f"#include <hip/hip_runtime.h>\n#include <{h}>\n" for h in HEADERS]
    with ThreadPoolExecutor(max_workers=6) as pool:
        results = list(pool.map(_syntax_only, sources))
    bad = [(h, out[-2000:]) for h, (rc, out) in zip(HEADERS, results) if rc != 0]
    assert not bad, bad


def test_mma_simt_namespace_compiles_against_the_reference_spelling():
    rc, out = _syntax_only(MMA_SIMT)
    assert rc == 0, out[-4000:]


def test_detail_names_of_the_reference_are_there():
    rc, out = _syntax_only(DETAIL_NAMES)
    assert rc == 0, out[-4000:]


@pytest.mark.parametrize("n", [8, -1])
def test_wait_group_rejects_what_it_cannot_count(n):
    src = ("#include <hip/hip_runtime.h>\n#include <wmma_extension/utils.hpp>\n"
           "__global__ void k() { mtk::wmma::utils::cp_async::wait_group<%d>(); }\n" % n)
    rc, out = _syntax_only(src)
    assert rc != 0 and "static assertion" in out

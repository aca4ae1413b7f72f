"""Writes tests/golden/primitive_kat.npz: the known-answer inputs the reference's
own primitive tests use, as plain arrays, with the dense matrices they stand for.

No file of the reference is read or executed; the values are the closed forms
its tests state:
  foreach_ij : src[i] = i/32 over a 16x16 tile         (test/primitive/foreach_ij.cu:104)
  map        : value i + j*M at (i,j)                  (test/primitive/map.cu:28)
  load_vector: v[i] = i/3, i < 16; the fragment must equal the load of a tile whose
               first 16 memory elements are v and the rest zero
                                                       (test/primitive/wmma.load_vector.cu:142-150)
  store_vector: src[i] = i over a 16x16 tile, the first 16 memory elements come back
                                                       (test/primitive/wmma.store_vector.cu:51-63)
  gevm       : 16x16 identity (1 where i % 17 == 0)     (test/primitive/gevm.cu:56)
  batch_gemm : A[j] = j/k, B[j] = j/n ramps             (test/tcec/batch_gemm.cu:507-513)
Run:  python tests/golden/make_fixtures.py
"""
import os

import numpy as np

M = 16
out = {}
out["foreach_ij_src"] = (np.arange(M * M, dtype=np.float32) / np.float32(32)).astype(np.float32)
ii, jj = np.meshgrid(np.arange(M), np.arange(M), indexing="ij")
out["map_value"] = (ii + jj * M).astype(np.float32)            # value stored at (i,j)
v = (np.arange(M, dtype=np.float32) / np.float32(3)).astype(np.float32)
out["load_vector_v"] = v
tile = np.zeros(M * M, dtype=np.float32)
tile[:M] = v
out["load_vector_tile"] = tile                                   # dense memory image
out["store_vector_src"] = np.arange(M * M, dtype=np.float32)
out["store_vector_expect"] = np.arange(M, dtype=np.float32)
eye = np.zeros(M * M, dtype=np.float32)
eye[np.arange(M * M) % 17 == 0] = 1
out["gevm_eye"] = eye
m = n = k = 64
out["bgemm_a"] = (np.arange(m * k, dtype=np.float32) / np.float32(k)).astype(np.float32)
out["bgemm_b"] = (np.arange(k * n, dtype=np.float32) / np.float32(n)).astype(np.float32)
# FP64 result of the reference's check loop for those ramps: c(i,j) = sum_l a[l + i*k] * b[l + j*k]
a64 = out["bgemm_a"].astype(np.float64).reshape(m, k)
b64 = out["bgemm_b"].astype(np.float64).reshape(n, k)
out["bgemm_c64"] = a64 @ b64.T                                    # (m,n)
# accuracy gates of the reference's one-warp tests (test/tcec/mma.cu:5-21)
out["threshold_with_ec"] = np.float64(1e-5)
out["threshold_without_ec"] = np.float64(1e-2)
np.savez(os.path.join(os.path.dirname(os.path.abspath(__file__)), "primitive_kat.npz"), **out)
print("wrote primitive_kat.npz")

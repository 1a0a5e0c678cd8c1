"""`from eed.backend import edgemm_m8n128k64x4, fastgemv, hgemm, ...` as the reference's scripts do
(script/standard-test.py:3-7, script/benchmark.py, script/gemv-test.py:3).

Every operator the reference declares (backend/cuda/hk/edgemm.h, flatgemm.h, edgemm_tr.h,
fastgemv.h, hgemm.h, backend/cuda/czn/fastgemm.h) is re-exported from the HIP extension.  A few
names in those scripts predate the current headers; the ones whose meaning is fixed by how the
scripts call them are aliased to the operator that took their place:

  edgemm_m8n32k128x8_bt(A, B_t, C)             -> gemm_m8n32k128x8_bt       (hk/edgemm_tr.cu:55-72)
  edgemm_m8n32k256x8_bt(A, B_t, C)             -> gemm_m8n32k256x8_bt       (hk/edgemm_tr.cu:99-116)
  edgemm_m8n64k128x8_bt_tuning(A, B_t, C, bz)  -> gemm_m8n64k128x8_bt_exp   (hk/edgemm_tr.cu:77-94)
  edgemm_m8n32k256x8_bt_tuning(A, B_t, C, bz)  -> gemm_m8n32k256x8_bt_bz2   (hk/edgemm_tr.cu:122-139)

Names with no surviving definition (edgemm_m8n128k64x8, hgemm_warp2, edgemm_mix, fastgemv_ex, ...)
are not guessed at: importing them raises ImportError, as it does against the reference's own
current sources.  There is no CPU fallback: without the built extension this import fails.
"""
from fastgate_amd import speedgate as _sg

_names = [n for n in dir(_sg) if not n.startswith("_")]
globals().update({n: getattr(_sg, n) for n in _names})

edgemm_m8n32k128x8_bt = _sg.gemm_m8n32k128x8_bt
edgemm_m8n32k256x8_bt = _sg.gemm_m8n32k256x8_bt
edgemm_m8n64k128x8_bt_tuning = _sg.gemm_m8n64k128x8_bt_exp
edgemm_m8n32k256x8_bt_tuning = _sg.gemm_m8n32k256x8_bt_bz2

__all__ = _names + ["edgemm_m8n32k128x8_bt", "edgemm_m8n32k256x8_bt", "edgemm_m8n64k128x8_bt_tuning",
                    "edgemm_m8n32k256x8_bt_tuning"]

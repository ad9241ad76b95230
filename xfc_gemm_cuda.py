"""Importable under the name the reference looks for (dl_base.py:26-32,
setup.py:8): `import xfc_gemm_cuda; xfc_gemm_cuda.xfc_gemm(in1, in2, out, alpha,
beta, apply_sigmoid)`."""
from renee_amd.xfc import xfc_gemm  # noqa: F401

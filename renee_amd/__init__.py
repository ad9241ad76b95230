"""MI355X-native XFC (extreme classifier) layer step: host interface over the
HIP library.  See include/xfc_mi355x.h for the C ABI."""
from .xfc import XFCLayer, coo_to_csr, xfc_gemm  # noqa: F401

"""MI355X-native XFC (extreme classifier) layer step: host interface over the
HIP library.  See include/xfc_mi355x.h for the C ABI."""
from .xfc import (XFCLayer, batch_positives, coo_to_csr, cosine_schedule_with_warmup,  # noqa: F401
                  read_sparse_labels, xfc_gemm)
from .loss import BCELossMultiNode  # noqa: F401
from .autograd import xfc_loss  # noqa: F401

"""MI355X-native policy-loss hot path of allenai/open-instruct.

The sub-modules carry the reference's own module and function names
(``model_utils.log_softmax_and_gather``, ``rl_utils.masked_mean``, ``grpo_utils.compute_grpo_loss``,
``padding_free_collator.get_batch_logps``, ``dpo_utils.dpo_loss`` ...), so a caller switches by
changing the import root.  Every function runs hand-written gfx950 HIP kernels through the
C-ABI in ``include/oi_kernels.h``; there is no CPU or eager-PyTorch fallback.
"""

from . import (  # noqa: F401
    _lib,
    data_loader,
    data_types,
    dpo_utils,
    grpo_utils,
    lm_head,
    model_utils,
    olmo_core_train_modules,
    olmo_core_utils,
    padding_free_collator,
    rl_utils,
)
from .grpo_utils import INVALID_LOGPROB  # noqa: F401
from .lm_head import fused_linear_cross_entropy, fused_lm_head_logprobs  # noqa: F401

__version__ = "0.1.0"

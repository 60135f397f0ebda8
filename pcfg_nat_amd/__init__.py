"""MI355X-native structured-loss ops of PCFG-NAT behind the reference's operator API
(``fs_plugins/custom_ops/__init__.py:1``)."""
from .custom_ops import (cuda_pcfg_loss, cuda_pcfg_best_tree, cuda_pcfg_viterbi, dag_logsoftmax_gather_inplace,
                         viterbi_decoding)

__all__ = ["cuda_pcfg_loss", "cuda_pcfg_best_tree", "cuda_pcfg_viterbi", "dag_logsoftmax_gather_inplace",
           "viterbi_decoding"]

"""MI355X-native DAG training operators for DA-Transformer (drop-in for fs_plugins/custom_ops)."""
from .custom_ops import (dag_loss, dag_best_alignment, dag_logsoftmax_gather_inplace,
                         torch_dag_loss, torch_dag_best_alignment, torch_dag_logsoftmax_gather_inplace)
from .custom_ops import dag_multihead_links, valid_end_from_tokens, valid_end_from_bound
from .custom_ops import dag_force_alignment, dag_glat_glance, dag_glat_oracle, dag_glat_mix
from .custom_ops import dag_viterbi_decode, dag_lookahead_decode, dag_logsoftmax_gather_argmax, dag_logsoftmax_max
from .custom_ops import dag_loss_float64_first
from .layouts import extract_valid_links, restore_valid_links, force_alignment

__all__ = ["dag_loss", "dag_best_alignment", "dag_logsoftmax_gather_inplace",
           "torch_dag_loss", "torch_dag_best_alignment", "torch_dag_logsoftmax_gather_inplace",
           "dag_multihead_links", "valid_end_from_tokens", "valid_end_from_bound",
           "dag_force_alignment", "dag_glat_glance", "dag_glat_oracle", "dag_glat_mix", "dag_viterbi_decode", "dag_lookahead_decode", "dag_logsoftmax_gather_argmax", "dag_logsoftmax_max", "dag_loss_float64_first",
           "extract_valid_links", "restore_valid_links", "force_alignment"]

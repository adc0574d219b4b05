"""MI355X-native DAG training operators for DA-Transformer (drop-in for fs_plugins/custom_ops)."""
from .custom_ops import (dag_loss, dag_best_alignment, dag_logsoftmax_gather_inplace,
                         torch_dag_loss, torch_dag_best_alignment, torch_dag_logsoftmax_gather_inplace)
from .layouts import extract_valid_links, restore_valid_links, force_alignment

__all__ = ["dag_loss", "dag_best_alignment", "dag_logsoftmax_gather_inplace",
           "torch_dag_loss", "torch_dag_best_alignment", "torch_dag_logsoftmax_gather_inplace",
           "extract_valid_links", "restore_valid_links", "force_alignment"]

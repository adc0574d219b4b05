from .dag_loss import (dag_loss, dag_best_alignment, dag_logsoftmax_gather_inplace, dag_logsoftmax_gather_argmax,
                       dag_logsoftmax_max, dag_loss_float64_first)
from .torch_ops import torch_dag_loss, torch_dag_best_alignment, torch_dag_logsoftmax_gather_inplace
from .links import dag_multihead_links, valid_end_from_tokens, valid_end_from_bound
from .glat import dag_force_alignment, dag_glat_glance, dag_glat_oracle, dag_glat_mix, GlatGlance
from .decode import dag_viterbi_decode, dag_lookahead_decode, ViterbiResult, LookaheadResult

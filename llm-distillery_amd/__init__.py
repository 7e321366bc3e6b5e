"""MI355X-native distillation-loss hot path of LLM-Distillery.

Hand-written gfx950 HIP kernels behind a C ABI (libdistill_hip.so), exposed
through the reference's own Python boundary (`calculate_divergence`, `Losses`).
"""
from . import _lib  # noqa: F401
from .batch_index import BatchIndex, ce_rows, content_rows, teachers_from_outgoing_batch  # noqa: F401
from .finetuning_utils import (LOSS_KEYS, calculate_divergence, distill_loss, distill_loss_batch,  # noqa: F401
                               distill_loss_batch_indexed)
from .h5_dataset import BatchPrefetcher, DistributionStore  # noqa: F401
from .losses import Losses  # noqa: F401
from .teacher_prep import fkl_multi_teacher, merge_remap_topk, merge_topk_pair, teacher_topk  # noqa: F401
from . import vocab_utils  # noqa: F401
from .ops import copy16, copy_rows, div_dense, div_topk, div_topk_static, reduce_sum, rowcoef_grad_topk, rowstats_topk  # noqa: F401

__all__ = ["BatchIndex", "LOSS_KEYS", "Losses", "calculate_divergence", "ce_rows", "content_rows", "copy16", "copy_rows", "distill_loss",
           "distill_loss_batch", "distill_loss_batch_indexed", "div_dense", "div_topk", "div_topk_static", "fkl_multi_teacher",
           "merge_remap_topk", "merge_topk_pair", "reduce_sum", "rowcoef_grad_topk", "rowstats_topk",
           "teacher_topk", "teachers_from_outgoing_batch", "vocab_utils"]

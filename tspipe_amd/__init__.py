"""MI355X-native teacher-student step kernels behind TSPipe's plug-in API.

Importing the package does not touch the GPU or the shared library; the
library is loaded on the first kernel call (see ``_lib``).
"""
from .batch_ops import (Batch, ScatterGatherFn, batch_size, check, defaultScatterGatherFn, gather,
                        generic_gather, generic_scatter, scatter, scatter_copy)
from .batchnorm import DeferredBatchNorm
from .ema import (bind_params_, calculate_target_network_parameters, calculate_updated_momentum_encoder,
                  clone_and_update, clone_params, copy_params_, momentum_update, update_target_network_parameters_)
from .losses import (Logits, SoftTarget, byol_contrastive_loss, byol_contrastive_loss_pieces, byol_loss, cosine_embedding_loss, cosine_embedding_loss_pieces, distil_ce_loss,
                     distil_loss_fn, distil_loss_fn_pieces, infonce_loss, kd_ce_loss, kd_ce_loss_pieces,
                     kd_soft_target_loss, logits_mse_loss, moco_contrastive_loss, moco_contrastive_loss_pair,
                     moco_contrastive_loss_pieces, set_infonce_fp32_arithmetic, set_infonce_workgroup_target,
                     soft_target_tspipe_loss)
from .model_wrapper import TSPipeModelOutput, TSPipeModelWrapper
from .utils import generic_object_gather, generic_object_scatter, traverse_tensor_map

__version__ = "0.1.0"

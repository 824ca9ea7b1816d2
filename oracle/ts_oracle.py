"""Eager PyTorch restatement of the reference's teacher-student step functions.

Test infrastructure (see the package docstring).  Every function works on CPU
tensors of any float dtype and follows the reference's op order, so that its
rounding is the reference's rounding.
"""
from collections import OrderedDict
from typing import Any, List, Optional, Sequence

import torch
import torch.nn.functional as F
from torch import Tensor, nn


# -- momentum EMA -------------------------------------------------------------

@torch.no_grad()
def ema_update(m: float, online_new_param: Sequence[Optional[Tensor]], target_param: Sequence[Tensor],
               skip_none: bool = False) -> List[Tensor]:
    """benchmarks/byol/trainer.py:198-212 (skip_none=False) and
    benchmarks/moco-v3/main.py:133-144 (skip_none=True): per tensor a clone of
    the teacher times m plus the student times the Python double (1. - m)."""
    result = []
    for param_q, param_k in zip(online_new_param, target_param):
        if param_q is None:
            if skip_none:
                continue
            raise TypeError("None student parameter")
        new = param_k.clone().detach()
        new = new * m + param_q.data * (1. - m)
        result.append(new)
    return result


# -- KD soft target -----------------------------------------------------------

def kd_soft_target(out_s: Tensor, out_t: Tensor, T: float) -> Tensor:
    """benchmarks/soft_target/kd_losses/st.py:18-23."""
    return F.kl_div(F.log_softmax(out_s / T, dim=1), F.softmax(out_t / T, dim=1),
                    reduction="batchmean") * T * T


def distil_ce(s_logits: Tensor, t_logits: Tensor, row_mask: Tensor, temperature: float,
              alpha_ce: float = 1.0) -> Tensor:
    """benchmarks/distilbert/distiller.py:719-740: masked_select with the row
    mask expanded over the vocabulary, KLDivLoss('batchmean') on the selected
    rows, times temperature squared and alpha_ce.  row_mask is [bs, seq] bool."""
    mask = row_mask.unsqueeze(-1).expand_as(s_logits)
    vocab = s_logits.size(-1)
    s_sel = torch.masked_select(s_logits, mask).view(-1, vocab)
    t_sel = torch.masked_select(t_logits, mask).view(-1, vocab)
    ce = nn.KLDivLoss(reduction="batchmean")(F.log_softmax(s_sel / temperature, dim=-1),
                                             F.softmax(t_sel / temperature, dim=-1)) * temperature ** 2
    return alpha_ce * ce


def logits_mse(out_s: Tensor, out_t: Tensor) -> Tensor:
    """benchmarks/soft_target/kd_losses/logits.py:17-20."""
    return F.mse_loss(out_s, out_t)


def soft_target_tspipe_loss(model_out: Tensor, ema_model_out: Tensor, label: Tensor, T: float,
                            lambda_kd: float, kd_mode: str = "st") -> Tensor:
    """benchmarks/soft_target/train_kd.py:439-453."""
    cls_loss = nn.CrossEntropyLoss()(model_out, label)
    if kd_mode == "logits":
        kd_loss = logits_mse(model_out, ema_model_out.detach()) * lambda_kd
    elif kd_mode == "st":
        kd_loss = kd_soft_target(model_out, ema_model_out.detach(), T) * lambda_kd
    else:
        assert False
    return cls_loss + kd_loss


def distil_loss(s_logits: Tensor, t_logits: Tensor, s_hidden: Optional[Tensor], t_hidden: Optional[Tensor],
                lm_labels: Tensor, attention_mask: Tensor, alpha_ce: float, alpha_mlm: float, alpha_cos: float,
                temperature: float, restrict_ce_to_mask: bool, alpha_clm: float = 0.0,
                alpha_mse: float = 0.0) -> Tensor:
    """benchmarks/distilbert/distiller.py:711-772: masked KD (719-740), masked-LM
    cross entropy with ignore_index=-100 (742-744, lm_loss_fct at 117),
    causal-LM cross entropy on shifted logits (745-749), sum-of-squares of the
    selected logits over their row count (751-755, mse_loss_fct at 119), cosine
    embedding loss on the last hidden states (756-770)."""
    mask2d = (lm_labels > -1) if restrict_ce_to_mask else attention_mask
    loss = distil_ce(s_logits, t_logits, mask2d, temperature, alpha_ce)
    if alpha_mlm > 0.0:
        loss_mlm = nn.CrossEntropyLoss(ignore_index=-100)(s_logits.view(-1, s_logits.size(-1)), lm_labels.view(-1))
        loss = loss + alpha_mlm * loss_mlm
    if alpha_clm > 0.0:
        shift_logits = s_logits[..., :-1, :].contiguous()
        shift_labels = lm_labels[..., 1:].contiguous()
        loss_clm = nn.CrossEntropyLoss(ignore_index=-100)(shift_logits.view(-1, shift_logits.size(-1)),
                                                          shift_labels.view(-1))
        loss = loss + alpha_clm * loss_clm
    if alpha_mse > 0.0:
        mask = mask2d.unsqueeze(-1).expand_as(s_logits)
        s_sel = torch.masked_select(s_logits, mask).view(-1, s_logits.size(-1))
        t_sel = torch.masked_select(t_logits, mask).view(-1, s_logits.size(-1))
        loss_mse = nn.MSELoss(reduction="sum")(s_sel, t_sel) / s_sel.size(0)
        loss = loss + alpha_mse * loss_mse
    if alpha_cos > 0.0:
        mask = attention_mask.unsqueeze(-1).expand_as(s_hidden)
        dim = s_hidden.size(-1)
        s_sel = torch.masked_select(s_hidden, mask).view(-1, dim)
        t_sel = torch.masked_select(t_hidden, mask).view(-1, dim)
        target = s_sel.new(s_sel.size(0)).fill_(1)
        loss_cos = nn.CosineEmbeddingLoss(reduction="mean")(s_sel, t_sel, target)
        loss = loss + alpha_cos * loss_cos
    return loss


# -- BYOL / MoCo --------------------------------------------------------------

def byol_regression_loss(x: Tensor, y: Tensor) -> Tensor:
    """benchmarks/byol/trainer.py:51-55."""
    x = F.normalize(x, dim=1)
    y = F.normalize(y, dim=1)
    return 2 - 2 * (x * y).sum(dim=-1)


def byol_contrastive_loss(o1: Tensor, o2: Tensor, t1: Tensor, t2: Tensor) -> Tensor:
    """benchmarks/byol/trainer.py:192-196."""
    loss = byol_regression_loss(o1, t2)
    loss = loss + byol_regression_loss(o2, t1)
    return loss.mean()


def infonce(q: Tensor, k: Tensor, tau: float) -> Tensor:
    """The inner ``loss(q, k)`` of benchmarks/moco-v3/main.py:149-160."""
    q = F.normalize(q, dim=1)
    k = F.normalize(k, dim=1)
    logits = torch.einsum("nc,mc->nm", [q, k]) / tau
    labels = torch.arange(logits.shape[0], dtype=torch.long).to(logits.device)  # main.py:155-157: built on the host, then moved
    return nn.CrossEntropyLoss()(logits, labels) * (2 * tau)


def moco_contrastive_loss(o1: Tensor, o2: Tensor, t1: Tensor, t2: Tensor, tau: float) -> Tensor:
    """benchmarks/moco-v3/main.py:162."""
    return infonce(o1, t2, tau) + infonce(o2, t1, tau)


# -- DeferredBatchNorm ----------------------------------------------------------

class DeferredBNOracle:
    """tspipe/batchnorm.py:24-120 as a plain object over CPU tensors."""

    def __init__(self, num_features: int, eps: float = 1e-5, momentum: Optional[float] = 0.1,
                 chunks: int = 1, weight: Optional[Tensor] = None, bias: Optional[Tensor] = None,
                 dtype=torch.float32):
        self.eps, self.momentum, self.chunks = eps, momentum, chunks
        self.weight, self.bias = weight, bias
        self.running_mean = torch.zeros(num_features, dtype=dtype)
        self.running_var = torch.ones(num_features, dtype=dtype)
        self.num_batches_tracked = torch.tensor(0, dtype=torch.long)
        self.sum = torch.zeros(num_features, dtype=dtype)
        self.sum_squares = torch.zeros(num_features, dtype=dtype)
        self.counter = 0
        self.tracked = 0
        self.training = True

    def track(self, x: Tensor) -> bool:
        """batchnorm.py:45-59."""
        dim = [0] + list(range(2, x.dim()))
        with torch.no_grad():
            self.sum += x.sum(dim)
            self.sum_squares += (x ** 2).sum(dim)
        self.counter += x.size().numel() // x.size(1)
        self.tracked += 1
        return self.tracked == self.chunks

    def commit(self) -> None:
        """batchnorm.py:61-85 (biased variance; in-place scale then add)."""
        self.num_batches_tracked += 1
        if self.momentum is None:
            factor = 1.0 / float(self.num_batches_tracked)
        else:
            factor = self.momentum
        mean = self.sum / self.counter
        var = self.sum_squares / self.counter - mean ** 2
        self.running_mean *= 1 - factor
        self.running_mean += mean * factor
        self.running_var *= 1 - factor
        self.running_var += var * factor
        self.sum.zero_()
        self.sum_squares.zero_()
        self.counter = 0
        self.tracked = 0

    def forward(self, x: Tensor) -> Tensor:
        """batchnorm.py:87-120."""
        if x.dim() <= 2:
            raise ValueError("expected at least 3D input (got %dD input)" % x.dim())
        if not self.training:
            return F.batch_norm(x, running_mean=self.running_mean, running_var=self.running_var,
                                weight=self.weight, bias=self.bias, training=False, momentum=0.0, eps=self.eps)
        if self.track(x):
            self.commit()
        return F.batch_norm(x, running_mean=None, running_var=None, weight=self.weight, bias=self.bias,
                            training=True, momentum=0.0, eps=self.eps)


# -- scatter / gather -----------------------------------------------------------

def scatter(value, chunks: int) -> list:
    """tspipe/batch_ops.py:168-183, returning bare tensors / tuples instead of Batch objects."""
    if isinstance(value, Tensor):
        return list(value.chunk(chunks))
    return list(zip(*[member.chunk(chunks) for member in value]))


def gather(pieces: list):
    """tspipe/batch_ops.py:186-205 over bare tensors / tuples."""
    if isinstance(pieces[0], Tensor):
        return torch.cat(tuple(pieces))
    return tuple(torch.cat(group) for group in zip(*pieces))


def generic_object_scatter(obj: Any, chunks: int, output_cls=None) -> Any:
    """tspipe/utils.py:225-254.  dict is matched before OrderedDict, as in the
    reference.  output_cls: the TSPipeModelOutput-like dataclass to unwrap and
    re-wrap at the top level (utils.py:246-250), if any."""
    if output_cls is not None and isinstance(obj, output_cls):
        return [output_cls(data=x, lst_require_grad_tensor_path=obj.lst_require_grad_tensor_path)
                for x in generic_object_scatter(obj.data, chunks)]
    if isinstance(obj, list):
        return [list(x) for x in zip(*[generic_object_scatter(x, chunks) for x in obj])]
    if isinstance(obj, tuple):
        return tuple(zip(*[generic_object_scatter(x, chunks) for x in obj]))
    if isinstance(obj, dict):
        keys = zip(*[generic_object_scatter(k, chunks) for k in obj.keys()])
        vals = zip(*[generic_object_scatter(v, chunks) for v in obj.values()])
        return tuple(dict(zip(*kv)) for kv in zip(keys, vals))
    if isinstance(obj, Tensor):
        return obj.chunk(chunks)
    return [obj for _ in range(chunks)]


def generic_object_gather(*objs: Any, output_cls=None) -> Any:
    """tspipe/utils.py:256-292.  With output_cls, a call whose arguments are all
    of that class gathers their .data and keeps the first one's path list; as in
    the reference, that test is vacuously true for an empty call, which then
    fails on objs[0]."""
    if output_cls is not None and all(isinstance(o, output_cls) for o in objs):
        return output_cls(data=generic_object_gather(*[o.data for o in objs]),
                          lst_require_grad_tensor_path=objs[0].lst_require_grad_tensor_path)
    if len(objs) == 0:
        return tuple()
    first = objs[0]
    if any(type(first) != type(o) for o in objs):
        raise ValueError("Type of given objects must match")
    if isinstance(first, list):
        return [generic_object_gather(*g) for g in zip(*objs)]
    if isinstance(first, (tuple, zip)):
        return tuple(generic_object_gather(*g) for g in zip(*objs))
    if isinstance(first, dict):
        for other in objs:
            if any(a != b for a, b in zip(first.keys(), other.keys())):
                raise ValueError("Key of given objects must match")
        items = [(g[0][0], generic_object_gather(*[kv[1] for kv in g])) for g in zip(*[o.items() for o in objs])]
        return OrderedDict(items) if isinstance(first, OrderedDict) else dict(items)
    if isinstance(first, Tensor):
        return torch.cat(objs)
    if any(first != o for o in objs):
        raise ValueError("Value of given objects must match")
    return first

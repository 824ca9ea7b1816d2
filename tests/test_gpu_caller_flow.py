"""The plug-ins driven the way TSPipe's GPU worker drives them.

A miniature teacher-student training loop restates what the reference's worker
does around its plug-ins, on one partition:

* forward (tspipe/gpu_task.py:431-532): a micro-batch is scattered once more
  into backward-sized pieces, every piece runs through the partition (the
  teacher's without gradients but in train mode, tspipe/tspipe.py:61,186-192),
  the piece outputs are gathered into the micro-batch's output and kept as
  activations;
* loss (tspipe/gpu_task.py:89-226): every student output is detached, scattered
  into the backward-sized pieces, made a gradient leaf with a hook that stores
  its gradient (structured outputs: only on paths that contain 'logits', 131-143),
  gathered again, then gathered over the micro-batches; ``loss_fn`` runs on the
  result and ``torch.autograd.backward`` fills the gradient store;
* backward: the stored gradients flow into the kept activations;
* optimize (tspipe/gpu_task.py:385-410): optimizer step, clone of the student
  parameters, ``target_update_fn(momentum, online_new_param, target_prev_param)``
  whose result is a NEW list;
* update (tspipe/gpu_task.py:706-724): ``param.copy_`` of that list into the teacher.

The loop runs twice on the same seeded data: on the GPU with this package's
plug-ins (DeferredBatchNorm converter, scatter/gather, loss, target update), and
on the CPU with the oracle's restatement of the reference's functions.  Losses,
student and teacher parameters and the BatchNorm buffers must agree after several
steps; tolerances are fp32 rounding accumulated over the steps (stated below).
"""
import copy
from argparse import Namespace
from functools import partial

import pytest
import torch
from torch import nn

import tspipe_amd as ta
from oracle import ts_oracle

from helpers import max_rel_to_peak, rel_err, seeded

pytestmark = pytest.mark.gpu

STEPS = 4
NUM_UBATCH = 2
MOMENTUM = 0.9          # teacher momentum; far from 1 so that a wrong update shows after 4 steps
REL_LOSS = 5e-6         # per-step loss, relative, times the step number (measured: up to 7e-7)
REL_PARAM = 2e-5        # final tensors, max |diff| / max |ref| (measured: up to 1.3e-6)


# ---- the two sets of plug-ins ----------------------------------------------------

class ProductPlugins:
    """What a TSPipe user passes in, taken from this package."""

    def __init__(self, structured: bool):
        self.sg = (ta.ScatterGatherFn(ta.generic_scatter, ta.generic_gather, ta.batch_size) if structured
                   else ta.defaultScatterGatherFn)
        self.output_cls = ta.TSPipeModelOutput

    def scatter(self, value, chunks):
        return [b.value for b in self.sg.scatter(value, chunks)]

    def gather(self, values):
        return self.sg.gather([ta.Batch(v) for v in values])

    def convert(self, module, chunks):
        return ta.DeferredBatchNorm.convert_deferred_batch_norm(module, chunks)

    def wrap(self, model):
        return ta.TSPipeModelWrapper(model)

    target_update = staticmethod(ta.calculate_target_network_parameters)

    @staticmethod
    def byol(o1, o2, t1, t2, args, extra):
        return ta.byol_contrastive_loss(o1, o2, t1, t2, args, extra)

    @staticmethod
    def moco(o1, o2, t1, t2, args, extra):
        return ta.moco_contrastive_loss(o1, o2, t1, t2, args, extra)

    @staticmethod
    def soft_target(s, t, label, tspipe_args, args, epoch):
        return ta.soft_target_tspipe_loss(s, t, label, tspipe_args, args, epoch)

    @staticmethod
    def distil(s, t, labels, tspipe_args, params, epoch):
        return ta.distil_loss_fn(s, t, labels, tspipe_args, params, epoch)


class _OracleOutput:
    """Carrier with the two fields of the reference's TSPipeModelOutput."""

    def __init__(self, data, lst_require_grad_tensor_path):
        self.data, self.lst_require_grad_tensor_path = data, lst_require_grad_tensor_path


class _OracleBN(nn.Module):
    """nn.Module shell around the oracle's DeferredBatchNorm object, sharing the
    affine parameters of the layer it replaces."""

    def __init__(self, bn, chunks):
        super().__init__()
        self.weight, self.bias = bn.weight, bn.bias
        self.o = ts_oracle.DeferredBNOracle(bn.num_features, bn.eps, bn.momentum, chunks, self.weight, self.bias)

    def forward(self, x):
        self.o.training = self.training
        return self.o.forward(x)


class _OracleWrapper(nn.Module):
    def __init__(self, model):
        super().__init__()
        self.model = model

    def forward(self, x):
        out = self.model.forward(x.data if isinstance(x, _OracleOutput) else x)
        return out if isinstance(out, torch.Tensor) else _OracleOutput(out, None)


class OraclePlugins:
    """The same roles filled by the CPU restatement of the reference."""

    def __init__(self, structured: bool):
        self.structured = structured
        self.output_cls = _OracleOutput

    def scatter(self, value, chunks):
        if self.structured:
            return list(ts_oracle.generic_object_scatter(value, chunks, output_cls=_OracleOutput))
        return ts_oracle.scatter(value, chunks)

    def gather(self, values):
        if self.structured and not isinstance(values[0], torch.Tensor):
            return ts_oracle.generic_object_gather(*values, output_cls=_OracleOutput)
        return ts_oracle.gather(values)

    def convert(self, module, chunks):
        for name, child in list(module.named_children()):
            if isinstance(child, nn.modules.batchnorm._BatchNorm):
                setattr(module, name, _OracleBN(child, chunks))
            else:
                self.convert(child, chunks)
        return module

    def wrap(self, model):
        return _OracleWrapper(model)

    @staticmethod
    def target_update(m, online_new, target_prev):
        return ts_oracle.ema_update(m, online_new, target_prev)

    @staticmethod
    def byol(o1, o2, t1, t2, args, extra):
        return ts_oracle.byol_contrastive_loss(o1, o2, t1, t2)

    @staticmethod
    def moco(o1, o2, t1, t2, args, extra):
        return ts_oracle.moco_contrastive_loss(o1, o2, t1, t2, extra.moco_t)

    @staticmethod
    def soft_target(s, t, label, tspipe_args, args, epoch):
        return ts_oracle.soft_target_tspipe_loss(s, t, label, args.T, args.lambda_kd)

    @staticmethod
    def distil(s, t, labels, tspipe_args, p, epoch):
        lm_labels, attention_mask = labels
        return ts_oracle.distil_loss(s["logits"], t["logits"], s["hidden_states"][-1], t["hidden_states"][-1],
                                     lm_labels, attention_mask, p.alpha_ce, p.alpha_mlm, p.alpha_cos,
                                     p.temperature, p.restrict_ce_to_mask, alpha_mse=p.alpha_mse)


# ---- miniature networks ----------------------------------------------------------

class ChannelMix(nn.Module):
    """[N, C, L] -> [N, C_out, L]: a kernel-size-1 convolution as one matrix product."""

    def __init__(self, c_in, c_out):
        super().__init__()
        self.weight = nn.Parameter(torch.randn(c_out, c_in) * c_in ** -0.5)

    def forward(self, x):
        return torch.einsum("oc,ncl->nol", self.weight, x)


class MeanOverLength(nn.Module):
    def forward(self, x):
        return x.mean(dim=2)


def encoder():
    return nn.Sequential(ChannelMix(6, 8), nn.BatchNorm1d(8), nn.ReLU(), ChannelMix(8, 8), nn.BatchNorm1d(8),
                         nn.ReLU(), MeanOverLength(), nn.Linear(8, 16))


def classifier():
    return nn.Sequential(ChannelMix(6, 8), nn.BatchNorm1d(8), nn.ReLU(), MeanOverLength(), nn.Linear(8, 10))


class TokenModel(nn.Module):
    """ids [N, L] -> {'logits': [N, L, V], 'hidden_states': (h0, h1)} like a masked-LM head."""

    def __init__(self, vocab=37, width=12):
        super().__init__()
        self.embed = nn.Embedding(vocab, width)
        self.mix = nn.Linear(width, width)
        self.head = nn.Linear(width, vocab)

    def forward(self, ids):
        h0 = self.embed(ids)
        h1 = torch.tanh(self.mix(h0))
        return {"logits": self.head(h1), "hidden_states": (h0, h1)}


# ---- the worker's flow -----------------------------------------------------------

def _paths_requiring_grad(obj):
    """Paths of the tensors inside a nested output that require gradients."""
    found = []

    def walk(o, path):
        if isinstance(o, (list, tuple)):
            for i, c in enumerate(o):
                walk(c, path + (i,))
        elif isinstance(o, dict):
            for k, v in o.items():
                walk(v, path + (k,))
        elif isinstance(o, torch.Tensor) and o.requires_grad:
            found.append(path)

    walk(obj, ())
    return found


def _at(obj, path):
    for key in path:
        obj = obj[key]
    return obj


def _detach(value, output_cls):
    if isinstance(value, output_cls):
        return output_cls(_detach(value.data, output_cls), value.lst_require_grad_tensor_path)
    if isinstance(value, torch.Tensor):
        return value.detach()
    if isinstance(value, dict):
        return {k: _detach(v, output_cls) for k, v in value.items()}
    if isinstance(value, (list, tuple)):
        return type(value)(_detach(v, output_cls) for v in value)
    return value


def forward_task(plug, partition, ubatch, bwd_split, is_target):
    """One forward task: returns the micro-batch's gathered output and, for the
    student, the per-piece outputs that stay behind as activations."""
    piece_outputs = []
    for piece in plug.scatter(ubatch, bwd_split):
        if is_target:
            with torch.no_grad():
                out = partition(piece)
        else:
            out = partition(piece)
            if isinstance(out, plug.output_cls):
                out.lst_require_grad_tensor_path = _paths_requiring_grad(out.data)
        piece_outputs.append(out)
    return plug.gather(piece_outputs), (None if is_target else piece_outputs)


def loss_task(plug, loss_fn, student_outputs, teacher_outputs, label, bwd_split):
    """The loss task over all micro-batches of one mini-batch.  student_outputs and
    teacher_outputs map a view id to the list of per-micro-batch outputs.  Returns
    the loss value and the gradient store {(view, backward piece): {path: grad}}."""
    store = {}

    def keep(grad, key, path):
        store.setdefault(key, {})[path] = grad

    collected = {}
    for view, outputs in student_outputs.items():
        collected[view] = []
        for ubatch_id, output in enumerate(outputs):
            pieces = plug.scatter(_detach(output, plug.output_cls), bwd_split)
            for idx, piece in enumerate(pieces):
                key = (view, bwd_split * ubatch_id + idx)
                if isinstance(piece, torch.Tensor):
                    piece.requires_grad = True
                    piece.register_hook(partial(keep, key=key, path=()))
                else:
                    for path in piece.lst_require_grad_tensor_path:
                        if "logits" in path:
                            leaf = _at(piece.data, path)
                            assert leaf.is_leaf and not leaf.requires_grad
                            leaf.requires_grad = True
                            leaf.register_hook(partial(keep, key=key, path=path))
            collected[view].append(plug.gather(pieces))

    def whole(per_ubatch):
        value = plug.gather(per_ubatch)
        return value.data if isinstance(value, plug.output_cls) else value

    teachers = {view: [_detach(o, plug.output_cls) for o in outs] for view, outs in teacher_outputs.items()}
    if label is not None:       # asymmetric: one view, labels (gpu_task.py:165-181)
        loss = loss_fn(whole(collected[0]), whole(teachers[0]), label, Namespace(), ARGS, 0)
    else:                       # symmetric: two views (gpu_task.py:183-203)
        loss = loss_fn(whole(collected[0]), whole(collected[1]), whole(teachers[0]), whole(teachers[1]),
                       Namespace(), ARGS)
    value = loss.detach().cpu().item()
    torch.autograd.backward(loss, grad_tensors=None)
    return value, store


def backward_tasks(activations, store):
    """Gradients from the store into the kept activations, last piece first."""
    for (view, piece_id) in sorted(store, reverse=True):
        out = activations[view][piece_id]
        for path, grad in store[(view, piece_id)].items():
            leaf = out if path == () else _at(out.data, path)
            torch.autograd.backward(leaf, grad_tensors=grad, retain_graph=True)


ARGS = Namespace(moco_t=0.2, T=4.0, lambda_kd=0.7, kd_mode="st", alpha_ce=5.0, alpha_mlm=2.0, alpha_clm=0.0,
                 alpha_mse=0.5, alpha_cos=1.0, temperature=2.0, restrict_ce_to_mask=True)


def train(plug, device, case, bwd_split):
    make, loss_name, data = CASES[case]
    torch.manual_seed(7)
    student = make()
    teacher = copy.deepcopy(student)
    for p in teacher.parameters():
        p.requires_grad_(False)
    if case == "distil":
        student, teacher = plug.wrap(student), plug.wrap(teacher)
    student = plug.convert(student, NUM_UBATCH).to(device)
    teacher = plug.convert(teacher, NUM_UBATCH).to(device)
    student.train()
    teacher.train()
    optimizer = torch.optim.SGD(student.parameters(), lr=0.05, momentum=0.9)
    loss_fn = getattr(plug, loss_name)
    g = seeded(11)
    losses = []
    for _ in range(STEPS):
        views, label = data(g)
        views = [v.to(device) for v in views]
        if label is not None:
            label = tuple(x.to(device) for x in label) if isinstance(label, tuple) else label.to(device)
        s_out, t_out, activations = {}, {}, {}
        for view, batch in enumerate(views):
            s_out[view], t_out[view], activations[view] = [], [], []
            for ubatch in plug.scatter(batch, NUM_UBATCH):
                gathered, kept = forward_task(plug, student, ubatch, bwd_split, False)
                s_out[view].append(gathered)
                activations[view].extend(kept)
        # the teacher sees the other view in the two-view losses; its outputs are indexed by the view it read
        for view, batch in enumerate(views):
            for ubatch in plug.scatter(batch, NUM_UBATCH):
                t_out[view].append(forward_task(plug, teacher, ubatch, bwd_split, True)[0])
        value, store = loss_task(plug, loss_fn, s_out, t_out, label, bwd_split)
        losses.append(value)
        backward_tasks(activations, store)
        # optimize + target update + copy into the live teacher
        online_prev = list(student.parameters())
        target_prev = list(teacher.parameters())
        optimizer.step()
        optimizer.zero_grad()
        online_new = [t.detach().clone() for t in online_prev]
        before = [t.detach().clone() for t in target_prev]
        target_new = plug.target_update(MOMENTUM, online_new, target_prev)
        assert all(a.data_ptr() != b.data_ptr() for a, b in zip(target_new, target_prev)), "result aliases the teacher"
        assert all(torch.equal(a, b) for a, b in zip(before, target_prev)), "teacher changed before the copy"
        with torch.no_grad():
            for p, new in zip(teacher.parameters(), target_new):
                p.copy_(new, non_blocking=True)
    state = {"student." + k: v for k, v in _named_state(student).items()}
    state.update({"teacher." + k: v for k, v in _named_state(teacher).items()})
    return losses, state


def _named_state(module):
    out = {k: v.detach().cpu() for k, v in module.named_parameters()}
    for name, child in module.named_modules():
        holder = child.o if isinstance(child, _OracleBN) else child if isinstance(child, ta.DeferredBatchNorm) else None
        if holder is not None:
            for buf in ("running_mean", "running_var", "num_batches_tracked", "sum", "sum_squares"):
                out[f"{name}.{buf}"] = getattr(holder, buf).detach().cpu()
            out[f"{name}.counter"] = torch.tensor(int(holder.counter))
            out[f"{name}.tracked"] = torch.tensor(int(holder.tracked))
    return out


def _two_views(g):
    return [torch.randn(16, 6, 10, generator=g) * 1.5 + 0.5, torch.randn(16, 6, 10, generator=g) * 1.5 + 0.5], None


def _labelled(g):
    return [torch.randn(16, 6, 10, generator=g)], torch.randint(0, 10, (16,), generator=g)


def _tokens(g):
    ids = torch.randint(0, 37, (8, 12), generator=g)
    lm_labels = torch.where(torch.rand(8, 12, generator=g) < 0.3, ids, torch.full_like(ids, -100))
    attention = torch.rand(8, 12, generator=g) < 0.9
    return [ids], (lm_labels, attention)


CASES = {
    "byol": (encoder, "byol", _two_views),
    "moco": (encoder, "moco", _two_views),
    "soft_target": (classifier, "soft_target", _labelled),
    "distil": (TokenModel, "distil", _tokens),
}


@pytest.mark.parametrize("case,bwd_split", [("byol", 1), ("moco", 2), ("soft_target", 2), ("distil", 1), ("distil", 2)])
def test_training_loop_with_the_plug_ins_follows_the_oracle_loop(device, case, bwd_split):
    structured = case == "distil"
    got_losses, got = train(ProductPlugins(structured), device, case, bwd_split)
    ref_losses, ref = train(OraclePlugins(structured), torch.device("cpu"), case, bwd_split)
    assert len(got_losses) == STEPS
    for step, (a, b) in enumerate(zip(got_losses, ref_losses)):
        assert rel_err(a, b) <= REL_LOSS * (step + 1), (case, step, a, b)
    assert ref_losses[-1] != ref_losses[0]
    assert set(got) == set(ref)
    for name in sorted(ref):
        if ref[name].dtype == torch.long:
            assert torch.equal(got[name], ref[name]), name
        else:
            assert max_rel_to_peak(got[name], ref[name]) <= REL_PARAM, (case, name)
    # the teacher moved, and not onto the student
    moved = [n for n in ref if n.startswith("teacher.") and ref[n].dtype != torch.long
             and n.replace("teacher.", "student.") in ref
             and not torch.equal(ref[n], ref[n.replace("teacher.", "student.")])]
    assert moved

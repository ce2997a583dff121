"""The native Adam operator under the names the reference imports it by.

``patrickstar/ops/fp16_cpu_adam.py:177-193`` loads a pybind module ``cpu_adam_op``
with ``create_adam``, ``adam_update`` and ``destroy_adam``
(``patrickstar/ops/csrc/adam/cpu_adam.cpp:751-756``).  These are the same three
functions with the same argument meaning, taking flat torch tensors; the
arithmetic runs on the GPU through ``ps_adam_create`` / ``ps_adam_update`` /
``ps_adam_destroy``.  Like the reference's, each returns 0; failures raise.
"""
import torch

from . import _lib


def create_adam(optimizer_id, alpha=1e-3, betta1=0.9, betta2=0.999, eps=1e-8, weight_decay=0.0, adamw_mode=True,
                should_log=False):
    _lib.check(
        _lib.load().ps_adam_create(optimizer_id, alpha, betta1, betta2, eps, weight_decay, int(bool(adamw_mode)),
                                   int(bool(should_log))),
        "create_adam",
    )
    return 0


def destroy_adam(optimizer_id):
    _lib.check(_lib.load().ps_adam_destroy(optimizer_id), "destroy_adam")
    return 0


def adam_update(optimizer_id, step, lr, beta1, beta2, epsilon, weight_decay, bias_correction, params, grads, exp_avg,
                exp_avg_sq, loss_scale):
    """One update of one flat tensor, in place on ``params``, ``exp_avg`` and ``exp_avg_sq``.

    ``params``, ``exp_avg``, ``exp_avg_sq``: 1-D contiguous float32 tensors on the GPU (the reference asserts
    CPU tensors here, ``fp16_cpu_adam.py:222-225``); ``grads``: float32 or float16, never written;
    ``loss_scale <= 0``: no unscale.
    """
    for name, t in (("params", params), ("grads", grads), ("exp_avg", exp_avg), ("exp_avg_sq", exp_avg_sq)):
        if not t.is_cuda:
            raise RuntimeError(f"adam_update: {name} must be a GPU tensor (got {t.device})")
        if t.dim() != 1 or not t.is_contiguous():
            raise RuntimeError(f"adam_update: {name} must be flat and contiguous (call .view(-1))")
    if params.dtype != torch.float or exp_avg.dtype != torch.float or exp_avg_sq.dtype != torch.float:
        raise TypeError("adam_update: params, exp_avg and exp_avg_sq must be float32")
    if grads.dtype not in (torch.float, torch.half):
        raise TypeError(f"adam_update: grads must be float32 or float16, got {grads.dtype}")
    n = params.size(0)
    if not (grads.size(0) == exp_avg.size(0) == exp_avg_sq.size(0) == n):
        raise RuntimeError("adam_update: tensors differ in length")
    with torch.cuda.device(params.device):
        _lib.check(
            _lib.load().ps_adam_update(
                optimizer_id, int(step), lr, beta1, beta2, epsilon, weight_decay, int(bool(bias_correction)),
                params.data_ptr(), grads.data_ptr(), int(grads.dtype == torch.half), exp_avg.data_ptr(),
                exp_avg_sq.data_ptr(), n, float(loss_scale), None, _lib.current_stream_handle(),
            ),
            "adam_update",
        )
    return 0

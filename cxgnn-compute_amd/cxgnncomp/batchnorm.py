"""Batch normalisation between the convolutions of the models.

The upstream models use ``torch.nn.BatchNorm1d`` followed by ``F.relu``
(cxgnncomp/model.py:28, :66-67).  ``BatchNorm1d`` here is that module (same
parameters, buffers, state dict and arithmetic) whose CUDA fp32 path for 2-D
inputs runs on the library's batch-norm kernels, with the ReLU optionally fused:
``bn(x, relu=True)`` equals ``F.relu(bn(x))``.  Other inputs take torch's path.
"""
import torch
import torch.nn.functional as F

from cxgnncomp_backend import _ops


class _BatchNormFunction(torch.autograd.Function):

    @staticmethod
    def forward(ctx, x, weight, bias, running_mean, running_var, factor, eps, relu):
        mean, invstd, var_unbiased = _ops.batchnorm_stats(x, eps)
        y = _ops.batchnorm_apply(x, mean, invstd, weight, bias, relu)
        if running_mean is not None:
            running_mean.lerp_(mean, factor)
            running_var.lerp_(var_unbiased, factor)
        ctx.save_for_backward(x, weight, bias, mean, invstd)
        ctx.relu = relu
        return y

    @staticmethod
    def backward(ctx, dy):
        x, weight, bias, mean, invstd = ctx.saved_tensors
        dx, dgamma, dbeta = _ops.batchnorm_bwd(x, dy.contiguous(), mean, invstd, weight, bias, ctx.relu)
        return (dx, dgamma if weight is not None else None, dbeta if bias is not None else None,
                None, None, None, None, None)


class BatchNorm1d(torch.nn.BatchNorm1d):

    def forward(self, x, relu=False):
        native = (x.is_cuda and x.dim() == 2 and x.dtype == torch.float32 and x.shape[0] > 0
                  and (self.weight is None or self.weight.dtype == torch.float32))
        batch_stats = self.training or self.running_mean is None
        if native and not batch_stats and torch.is_grad_enabled() and (
                x.requires_grad or (self.weight is not None and self.weight.requires_grad)):
            native = False                    # gradients through the running statistics: torch's path
        if not native:
            out = super().forward(x)
            return F.relu(out) if relu else out
        x = x.contiguous()
        if not batch_stats:
            invstd = torch.rsqrt(self.running_var + self.eps)
            return _ops.batchnorm_apply(x, self.running_mean, invstd, self.weight, self.bias, relu)
        if x.shape[0] == 1:
            raise ValueError("Expected more than 1 value per channel when training, got input size %s"
                             % (tuple(x.shape),))
        # the running-average factor, as torch.nn.modules.batchnorm._BatchNorm.forward computes it
        factor = 0.0 if self.momentum is None else self.momentum
        update = self.training and self.track_running_stats
        if update and self.num_batches_tracked is not None:
            self.num_batches_tracked.add_(1)
            if self.momentum is None:
                factor = 1.0 / float(self.num_batches_tracked)
        return _BatchNormFunction.apply(x, self.weight, self.bias, self.running_mean if update else None,
                                        self.running_var if update else None, factor, self.eps, relu)

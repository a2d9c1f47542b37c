"""torch.nn.BatchNorm1d on (rows, C) feature matrices with an optional fused ReLU, on HIP
kernels (same parameters, buffers and state_dict keys as BatchNorm1d).  What the reference
builds from BatchNorm1d + ReLU(inplace) after every convolution
(ocnn/modules/modules.py:32-99, 120-153)."""

import torch
import torch.nn

from .. import _lib


def _param(t):
  """A per-channel parameter as the kernels read it (f32 / f16 / bf16, contiguous)."""
  if t is None:
    return None
  t = t.detach()
  if t.dtype not in _lib.DTYPE_CODE:
    t = t.float()
  return t.contiguous()


class _BatchNormRelu(torch.autograd.Function):
  @staticmethod
  def forward(ctx, x, weight, bias, running_mean, running_var, use_batch_stats, factor, eps, relu,
              residual=None, batches_tracked=None):
    L = _lib.lib()
    x = x.contiguous()
    rows, c = x.shape
    code = _lib.dtype_code(x)
    dev = x.device
    gamma, beta = _param(weight), _param(bias)
    if beta is not None and gamma is not None and beta.dtype != gamma.dtype:
      beta = beta.to(gamma.dtype)
    pcode = _lib.DTYPE_CODE[(gamma if gamma is not None else beta).dtype] if (gamma is not None or beta is not None) else 0
    if use_batch_stats:
      mean = torch.empty(c, dtype=torch.float32, device=dev)
      var = torch.empty(c, dtype=torch.float32, device=dev)
      invstd = torch.empty(c, dtype=torch.float32, device=dev)
      ws = _lib.workspace(L.ocnn_batch_norm_workspace_bytes(c), dev)
      track = running_mean is not None and factor is not None
      in_place = track and running_mean.dtype in _lib.DTYPE_CODE and running_mean.dtype == running_var.dtype \
          and running_mean.is_contiguous() and running_var.is_contiguous()
      _lib.check(L.ocnn_batch_norm_stats(
          code, _lib.ptr(x), rows, c, float(eps), _lib.ptr(mean), _lib.ptr(var), _lib.ptr(invstd),
          _lib.ptr(running_mean) if in_place else None, _lib.ptr(running_var) if in_place else None,
          _lib.DTYPE_CODE[running_mean.dtype] if in_place else 0, float(factor) if in_place else 0.0,
          _lib.ptr(batches_tracked), _lib.ptr(ws), ws.numel(), _lib.stream()))
      if track and not in_place:
        unbiased = var * (rows / max(rows - 1, 1))
        running_mean.mul_(1 - factor).add_(mean.to(running_mean.dtype), alpha=factor)
        running_var.mul_(1 - factor).add_(unbiased.to(running_var.dtype), alpha=factor)
    else:
      assert batches_tracked is None
      mean = running_mean.detach().float().contiguous()
      invstd = torch.rsqrt(running_var.detach().float() + eps)
    y = torch.empty_like(x)
    if residual is not None:
      residual = residual.contiguous()
      assert residual.shape == x.shape and residual.dtype == x.dtype
    _lib.check(L.ocnn_batch_norm_apply(code, _lib.ptr(x), rows, c, _lib.ptr(mean), _lib.ptr(invstd),
                                       _lib.ptr(gamma), _lib.ptr(beta), pcode, int(relu), _lib.ptr(residual),
                                       _lib.ptr(y), _lib.stream()))
    # with a residual the ReLU's mask is not a function of x alone: the output is kept for it
    ctx.save_for_backward(x, mean, invstd, gamma, beta, y if (residual is not None and relu) else None)
    ctx.has_residual = residual is not None
    ctx.relu, ctx.training, ctx.pcode = relu, use_batch_stats, pcode
    ctx.wdtype = None if weight is None else weight.dtype
    ctx.bdtype = None if bias is None else bias.dtype
    return y

  @staticmethod
  def backward(ctx, dy):
    L = _lib.lib()
    x, mean, invstd, gamma, beta, y = ctx.saved_tensors
    dy = dy.contiguous()
    rows, c = x.shape
    dev = x.device
    dgamma = torch.empty(c, dtype=torch.float32, device=dev)
    dbeta = torch.empty(c, dtype=torch.float32, device=dev)
    want_res = ctx.has_residual and ctx.needs_input_grad[9]
    dx = torch.empty_like(x) if (ctx.needs_input_grad[0] or want_res) else None
    dres = torch.empty_like(x) if want_res else None
    # the parameter gradients come out in the parameters' dtype where the kernels hold it
    gw = gb = None
    if gamma is not None and ctx.needs_input_grad[1] and ctx.wdtype == gamma.dtype:
      gw = torch.empty(c, dtype=gamma.dtype, device=dev)
    if beta is not None and ctx.needs_input_grad[2] and ctx.bdtype == beta.dtype and \
        (gamma is None or beta.dtype == gamma.dtype):
      gb = torch.empty(c, dtype=beta.dtype, device=dev)
    ws = _lib.workspace(L.ocnn_batch_norm_workspace_bytes(c), dev)
    _lib.check(L.ocnn_batch_norm_backward(
        _lib.dtype_code(x), _lib.ptr(x), _lib.ptr(dy), rows, c, _lib.ptr(mean), _lib.ptr(invstd), _lib.ptr(gamma),
        _lib.ptr(beta), ctx.pcode, int(ctx.relu), int(ctx.training), _lib.ptr(y), _lib.ptr(dx), _lib.ptr(dres),
        _lib.ptr(dgamma), _lib.ptr(dbeta), _lib.ptr(gw), _lib.ptr(gb), _lib.ptr(ws), ws.numel(), _lib.stream()))
    if gw is None and ctx.wdtype is not None and ctx.needs_input_grad[1]:
      gw = dgamma.to(ctx.wdtype)
    if gb is None and ctx.bdtype is not None and ctx.needs_input_grad[2]:
      gb = dbeta.to(ctx.bdtype)
    return dx, gw, gb, None, None, None, None, None, None, dres, None


class BatchNormRelu1d(torch.nn.BatchNorm1d):
  """BatchNorm1d [+ ReLU] in one pass over (rows, C) inputs on the GPU.  Inputs the kernels do
  not take (3-D, channel counts that are not a multiple of 16 bytes, a single row, tensors
  that are not on the GPU) go through torch.nn.BatchNorm1d itself, followed by a ReLU."""

  def __init__(self, num_features: int, relu: bool = False, **kwargs):
    super().__init__(num_features, **kwargs)
    self.fused_relu = relu

  def forward(self, input: torch.Tensor, residual: torch.Tensor = None, relu: bool = None) -> torch.Tensor:
    """residual: added to the normalised values before the ReLU (the tail of a residual
    block), in the same pass.  relu: overrides the module's setting for this call."""
    relu = self.fused_relu if relu is None else relu
    code = _lib.DTYPE_CODE.get(input.dtype, -1)
    if not (input.dim() == 2 and input.is_cuda and code >= 0 and input.shape[0] > 1 and
            _lib.lib().ocnn_batch_norm_supported(code, input.shape[0], input.shape[1])):
      out = super().forward(input)
      if residual is not None:
        out = out + residual
      return torch.relu(out) if relu else out
    # the bookkeeping of torch.nn.modules.batchnorm._BatchNorm.forward
    factor = 0.0 if self.momentum is None else self.momentum
    counter = None
    if self.training and self.track_running_stats and self.num_batches_tracked is not None:
      nbt = self.num_batches_tracked
      if (self.momentum is not None and nbt.is_cuda and nbt.dtype == torch.long and nbt.device == input.device):
        counter = nbt                        # counted by the statistics kernel: no launch of its own
      else:
        nbt.add_(1)
        factor = 1.0 / float(nbt) if self.momentum is None else self.momentum
    use_batch_stats = self.training or (self.running_mean is None and self.running_var is None)
    track = self.training and self.track_running_stats
    return _BatchNormRelu.apply(input, self.weight, self.bias,
                                self.running_mean if (not use_batch_stats or track) else None,
                                self.running_var if (not use_batch_stats or track) else None,
                                use_batch_stats, factor if track else None, self.eps, relu, residual, counter)

  def extra_repr(self) -> str:
    return super().extra_repr() + ', relu={}'.format(self.fused_relu)

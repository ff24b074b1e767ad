"""Synapse layers on time-innermost tensors: dense, convolution, pooling and their transposed forms.

Interface of lava.lib.dl.slayer.synapse.Conv (synapse/layer.py:178-323 in the reference): a spatial convolution
applied at every time step of an NCHWT tensor.  The reference calls ``F.conv3d`` with a kernel of (kh, kw, 1); the
library behind it wants channels last and transposes the tensor there and back around its kernel.  Here
slayer_conv_synapse of libslayer_hip.so computes it where the tensor lies, so the neuron that follows reads the
result in place; the input gradient is the same kernel on the flipped, transposed weights and the weight gradient
slayer_conv_synapse_wgrad.  What the kernels do not take (grouped convolutions, fewer than four time steps, more than
about 860 taps) goes to ``F.conv3d`` and its gradients as before.  The transposed convolution
(synapse/layer.py:511-658) and the unpooling layer (:661-838) are the same three kernels with their roles exchanged.
"""
import torch
import torch.nn.functional as F

from .. import _native as N

_ERANGE = -3


def _pair(v, what):
    if isinstance(v, int):
        return (v, v)
    if len(v) == 2:
        return (int(v[0]), int(v[1]))
    raise Exception(f'{what} can be either int or tuple of size 2. Found {v}')


def _launch(input, weight4, stride, padding, dilation):
    """out or None (None: outside what the kernel takes).  weight4: [Co, Ci, kh, kw]."""
    n, ci, h, w, t = input.shape
    co, _, kh, kw = weight4.shape
    ho = (h + 2 * padding[0] - dilation[0] * (kh - 1) - 1) // stride[0] + 1
    wo = (w + 2 * padding[1] - dilation[1] * (kw - 1) - 1) // stride[1] + 1
    if ho < 1 or wo < 1:
        raise RuntimeError(f'convolution kernel {kh}x{kw} does not fit an image of {h}x{w}')
    out = torch.empty((n, co, ho, wo, t), dtype=torch.float32, device=input.device)
    with N.device_guard(input.device):
        code = N.lib().slayer_conv_synapse(N.ptr(out), N.ptr(input), N.ptr(weight4), n, ci, co, h, w, t, kh, kw,
                                           stride[0], stride[1], padding[0], padding[1], dilation[0], dilation[1],
                                           N.stream_handle())
    if code == _ERANGE:
        return None
    N.check(code)
    return out


def _launch_input_grad(grad_output, weight_t4, input_shape, stride, padding, dilation):
    """Gradient of the input for any stride, or None (None: outside what the kernel takes).
    weight_t4: [Ci, Co, kh, kw], the forward weights with the channel axes exchanged."""
    n, ci, h, w, t = input_shape
    _, co, kh, kw = weight_t4.shape
    grad = torch.empty(tuple(input_shape), dtype=torch.float32, device=grad_output.device)
    with N.device_guard(grad_output.device):
        code = N.lib().slayer_conv_synapse_input_grad(N.ptr(grad), N.ptr(grad_output), N.ptr(weight_t4), n, ci, co, h, w,
                                                      t, kh, kw, stride[0], stride[1], padding[0], padding[1],
                                                      dilation[0], dilation[1], N.stream_handle())
    if code == _ERANGE:
        return None
    N.check(code)
    return grad


class _ConvSynapse(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, weight, stride, padding, dilation):
        out = _launch(input, weight.detach()[..., 0].contiguous(), stride, padding, dilation)
        if out is None:
            raise RuntimeError('not a shape the kernel takes')       # conv_synapse() checks before it gets here
        ctx.save_for_backward(input, weight)
        ctx.cfg = (stride, padding, dilation)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        input, weight = ctx.saved_tensors
        stride, padding, dilation = ctx.cfg
        grad_output = grad_output.contiguous()
        grad_input = grad_weight = None
        if ctx.needs_input_grad[0]:
            kh, kw = weight.shape[2], weight.shape[3]
            if stride == (1, 1):
                # the same convolution on the gradient, weights transposed and flipped
                flipped = weight.detach()[..., 0].flip(2, 3).transpose(0, 1).contiguous()
                back = (dilation[0] * (kh - 1) - padding[0], dilation[1] * (kw - 1) - padding[1])
                if back[0] >= 0 and back[1] >= 0:
                    grad_input = _launch(grad_output, flipped, (1, 1), back, dilation)
            if grad_input is None or grad_input.shape != input.shape:
                # any stride: the transposed form of the kernel
                grad_input = _launch_input_grad(grad_output, weight.detach()[..., 0].transpose(0, 1).contiguous(),
                                                input.shape, stride, padding, dilation)
            if grad_input is None:
                grad_input = torch.nn.grad.conv3d_input(input.shape, weight, grad_output, stride + (1,),
                                                        padding + (0,), dilation + (1,), 1)
        if ctx.needs_input_grad[1]:
            grad_weight = _weight_gradient(input, weight.shape, grad_output, stride, padding, dilation)
            if grad_weight is None:
                grad_weight = torch.nn.grad.conv3d_weight(input, weight.shape, grad_output, stride + (1,),
                                                          padding + (0,), dilation + (1,), 1)
        return grad_input, grad_weight, None, None, None


def _weight_gradient(input, weight_shape, grad_output, stride, padding, dilation):
    """[Co, Ci, kh, kw, 1] gradient of the weights or None (None: outside what the kernel takes)."""
    n, ci, h, w, t = input.shape
    co, _, kh, kw, _ = weight_shape
    lib = N.lib()
    floats = lib.slayer_conv_synapse_wgrad_workspace(n, ci, co, h, w, t, kh, kw, stride[0], padding[0], dilation[0])
    if floats == _ERANGE:
        return None
    if floats < 0:
        N.check(int(floats))
    grad = torch.empty((co, ci, kh, kw, 1), dtype=torch.float32, device=input.device)
    workspace = torch.empty(max(int(floats), 4), dtype=torch.float32, device=input.device)
    with N.device_guard(input.device):
        code = lib.slayer_conv_synapse_wgrad(N.ptr(grad), N.ptr(grad_output), N.ptr(input), n, ci, co, h, w, t, kh, kw,
                                             stride[0], stride[1], padding[0], padding[1], dilation[0], dilation[1],
                                             N.ptr(workspace), workspace.numel(), N.stream_handle())
    if code == _ERANGE:
        return None
    N.check(code)
    return grad


def conv_synapse(input, weight, stride=1, padding=0, dilation=1, groups=1):
    """``F.conv3d(input, weight, None, stride + (1,), padding + (0,), dilation + (1,), groups)`` for an NCHWT
    ``input`` and a ``weight`` of [Co, Ci / groups, kh, kw, 1], computed in place of the layout when the kernel
    takes the shape (one group, float32 on the GPU, at least four time steps), by the library call otherwise."""
    stride, padding, dilation = _pair(stride, 'stride'), _pair(padding, 'padding'), _pair(dilation, 'dilation')
    takes = (groups == 1 and input.is_cuda and input.dtype == torch.float32 and weight.dtype == torch.float32
             and input.dim() == 5 and weight.dim() == 5 and weight.shape[-1] == 1 and input.shape[-1] >= 4
             and input.shape[1] * weight.shape[2] * weight.shape[3] <= 860 and input.numel() > 0
             and input[0].numel() * 4 < 2 ** 31)
    if takes:
        input = input.contiguous()
    if not takes:
        return F.conv3d(input, weight, None, stride + (1,), padding + (0,), dilation + (1,), groups)
    return _ConvSynapse.apply(input, weight, stride, padding, dilation)


class _ConvTransposeSynapse(torch.autograd.Function):
    """The transposed convolution is the input gradient of a convolution from its output channels back to its
    input channels, so its three passes are that convolution's three kernels with their roles exchanged."""

    @staticmethod
    def forward(ctx, input, weight, stride, padding, dilation):
        n, _, h, w, t = input.shape
        _, co, kh, kw, _ = weight.shape
        shape = (n, co, (h - 1) * stride[0] - 2 * padding[0] + dilation[0] * (kh - 1) + 1,
                 (w - 1) * stride[1] - 2 * padding[1] + dilation[1] * (kw - 1) + 1, t)
        out = _launch_input_grad(input, weight.detach()[..., 0].transpose(0, 1).contiguous(), shape, stride, padding,
                                 dilation)
        if out is None:                                              # a limit conv_transpose_synapse() does not know
            out = F.conv_transpose3d(input, weight.detach(), None, stride + (1,), padding + (0,), 0, 1, dilation + (1,))
        ctx.save_for_backward(input, weight)
        ctx.cfg = (stride, padding, dilation)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        input, weight = ctx.saved_tensors
        stride, padding, dilation = ctx.cfg
        grad_output = grad_output.contiguous()
        grad_input = grad_weight = None
        if ctx.needs_input_grad[0]:
            grad_input = _launch(grad_output, weight.detach()[..., 0].contiguous(), stride, padding, dilation)
            if grad_input is None:
                grad_input = F.conv3d(grad_output, weight, None, stride + (1,), padding + (0,), dilation + (1,))
        if ctx.needs_input_grad[1]:
            # the weights of the convolution that runs backwards: its input is this layer's output
            grad_weight = _weight_gradient(grad_output, weight.shape, input, stride, padding, dilation)
            if grad_weight is None:
                grad_weight = torch.nn.grad.conv3d_weight(grad_output, weight.shape, input, stride + (1,),
                                                          padding + (0,), dilation + (1,), 1)
        return grad_input, grad_weight, None, None, None


def conv_transpose_synapse(input, weight, stride=1, padding=0, dilation=1, groups=1):
    """``F.conv_transpose3d(input, weight, None, stride + (1,), padding + (0,), 0, groups, dilation + (1,))`` for an
    NCHWT ``input`` and a ``weight`` of [Ci, Co / groups, kh, kw, 1], computed in place of the layout when the
    kernels take the shape (one group, float32 on the GPU, at least four time steps, strides up to 16), by the
    library call otherwise."""
    stride, padding, dilation = _pair(stride, 'stride'), _pair(padding, 'padding'), _pair(dilation, 'dilation')
    takes = (groups == 1 and input.is_cuda and input.dtype == torch.float32 and weight.dtype == torch.float32
             and input.dim() == 5 and weight.dim() == 5 and weight.shape[-1] == 1 and input.shape[-1] >= 4
             and input.numel() > 0 and max(stride) <= 16)
    if takes:
        _, co, kh, kw, _ = weight.shape
        ho = (input.shape[2] - 1) * stride[0] - 2 * padding[0] + dilation[0] * (kh - 1) + 1
        wo = (input.shape[3] - 1) * stride[1] - 2 * padding[1] + dilation[1] * (kw - 1) + 1
        takes = (0 < ho <= 60000 and 0 < wo <= 60000 and input.shape[1] * kh * kw <= 4096
                 and max(input[0].numel(), co * ho * wo * input.shape[-1]) * 4 < 2 ** 31)
    if not takes:
        return F.conv_transpose3d(input, weight, None, stride + (1,), padding + (0,), 0, groups, dilation + (1,))
    return _ConvTransposeSynapse.apply(input.contiguous(), weight, stride, padding, dilation)


class _SynapseLayer:
    """What the synapse layers share (GenericLayer, synapse/layer.py:15-69 in the reference): weight
    normalisation on demand, a pre-hook applied to the weight before every forward pass, ``shape``."""

    def _finish(self, weight_scale, weight_norm, pre_hook_fx):
        if weight_scale != 1:
            self.weight = torch.nn.Parameter(weight_scale * self.weight)
        self._pre_hook_fx = pre_hook_fx
        self.weight_norm_enabled = False
        self.complex = False
        if weight_norm is True:
            self.enable_weight_norm()

    def enable_weight_norm(self):
        torch.nn.utils.weight_norm(self, name='weight')
        self.weight_norm_enabled = True

    def disable_weight_norm(self):
        torch.nn.utils.remove_weight_norm(self, name='weight')
        self.weight_norm_enabled = False

    @property
    def grad_norm(self):
        """Norm of the weight gradient over its number of elements (0 before any backward pass)."""
        grad = (self.weight_g if self.weight_norm_enabled else self.weight).grad
        return 0 if grad is None else torch.norm(grad).item() / torch.numel(grad)

    @property
    def pre_hook_fx(self):
        return self._pre_hook_fx

    @pre_hook_fx.setter
    def pre_hook_fx(self, fx):
        self._pre_hook_fx = fx

    @property
    def shape(self):
        return self.weight.shape

    def _weight(self):
        return self.weight if self._pre_hook_fx is None else self._pre_hook_fx(self.weight)


class Dense(torch.nn.Conv3d, _SynapseLayer):
    """Dense synapse layer (synapse/layer.py:72-175 in the reference): every output neuron sums all input
    neurons of the same time step.  The reference writes it as ``F.conv3d`` with a kernel that covers the whole
    input; it is a matrix product of the [out, in] weights with the [N, in, T] spikes, and that is what runs
    here (``torch.matmul``: one batched GEMM whose result is time innermost, which the neuron kernels read in
    place).

    Parameters
    ----------
    in_neurons : int or (width, height) or (width, height, channels)
    out_neurons : int
    weight_scale, weight_norm, pre_hook_fx : as for :class:`Conv`.
    """

    def __init__(self, in_neurons, out_neurons, weight_scale=1, weight_norm=False, pre_hook_fx=None):
        if type(in_neurons) == int:
            kernel, in_channels = (1, 1, 1), in_neurons
        elif len(in_neurons) == 2:
            kernel, in_channels = (in_neurons[1], in_neurons[0], 1), 1
        elif len(in_neurons) == 3:
            kernel, in_channels = (in_neurons[1], in_neurons[0], 1), in_neurons[2]
        else:
            raise Exception(f'in_neurons should not be more than 3 dimension. Found {in_neurons=}')
        if type(out_neurons) != int:
            raise Exception(f'out_neurons should not be more than 1 dimension. Found {out_neurons=}')
        super().__init__(in_channels, out_neurons, kernel, bias=False)
        self._finish(weight_scale, weight_norm, pre_hook_fx)

    def forward(self, input):
        """Weighted spikes for NCT spikes ([N, out, T]) or NCHWT spikes ([N, out, 1, 1, T] when the image is the
        size of the kernel, the sliding convolution otherwise)."""
        weight = self._weight()
        if input.dim() == 3:
            return torch.matmul(weight.reshape(weight.shape[0], -1), input)
        if tuple(input.shape[1:4]) == tuple(weight.shape[1:4]):
            n, t = input.shape[0], input.shape[-1]
            return torch.matmul(weight.reshape(weight.shape[0], -1), input.reshape(n, -1, t)).reshape(n, -1, 1, 1, t)
        return F.conv3d(input, weight, self.bias, self.stride, self.padding, self.dilation, self.groups)


class Conv(torch.nn.Conv3d, _SynapseLayer):
    """Convolution synapse layer (synapse/layer.py:178-323 in the reference).

    Parameters
    ----------
    in_features, out_features : int
    kernel_size, stride, padding, dilation : int or (height, width)
    groups : int
    weight_scale : int
        weight initialization scale factor.
    weight_norm : bool
        weight normalization (``torch.nn.utils.weight_norm`` over the output channels, as in the reference).
    pre_hook_fx : callable or None
        applied to the weight before every forward pass (typically a quantizer).
    """

    def __init__(self, in_features, out_features, kernel_size, stride=1, padding=0, dilation=1, groups=1,
                 weight_scale=1, weight_norm=False, pre_hook_fx=None):
        kernel = _pair(kernel_size, 'kernel_size')
        self._stride2, self._padding2, self._dilation2 = _pair(stride, 'stride'), _pair(padding, 'padding'), \
            _pair(dilation, 'dilation')
        super().__init__(in_features, out_features, kernel + (1,), self._stride2 + (1,), self._padding2 + (0,),
                         self._dilation2 + (1,), groups, bias=False)
        self._finish(weight_scale, weight_norm, pre_hook_fx)

    def forward(self, input):
        """Weighted spikes [N, out_features, Ho, Wo, T] for spikes [N, in_features, H, W, T]."""
        return conv_synapse(input, self._weight(), self._stride2, self._padding2, self._dilation2, self.groups)


class Pool(torch.nn.Conv3d, _SynapseLayer):
    """Pooling synapse layer (synapse/layer.py:326-510 in the reference): every channel is summed over windows of
    ``kernel_size`` with a common weight (``weight_scale``, not trained).  The reference folds the channels into
    the image height and applies a one-channel ``F.conv3d``; here the same tensor goes through the convolution
    kernels of this package, its gradient through their transposed form.

    Parameters
    ----------
    kernel_size, stride, padding, dilation : int or (height, width); ``stride`` defaults to ``kernel_size``.
    weight_scale, weight_norm, pre_hook_fx : as for :class:`Conv`.
    """

    def __init__(self, kernel_size, stride=None, padding=0, dilation=1, weight_scale=1, weight_norm=False,
                 pre_hook_fx=None):
        kernel = _pair(kernel_size, 'kernel_size')
        self._stride2 = kernel if stride is None else _pair(stride, 'stride')
        self._padding2, self._dilation2 = _pair(padding, 'padding'), _pair(dilation, 'dilation')
        super().__init__(1, 1, kernel + (1,), self._stride2 + (1,), self._padding2 + (0,), self._dilation2 + (1,),
                         bias=False)
        self.weight = torch.nn.Parameter(weight_scale * torch.ones_like(self.weight), requires_grad=False)
        self._finish(1, weight_norm, pre_hook_fx)

    def forward(self, input):
        """Pooled spikes [N, C, Ho, Wo, T] for spikes [N, C, H, W, T]."""
        kh, kw = self.weight.shape[2], self.weight.shape[3]
        # as the reference does it: H % kh (W % kw) rows (columns) of zeros behind an image that is not a whole
        # number of windows, then the channels folded into the height
        if input.shape[2] % kh != 0:
            input = torch.cat((input, input.new_zeros(input.shape[0], input.shape[1], input.shape[2] % kh,
                                                      input.shape[3], input.shape[4])), 2)
        if input.shape[3] % kw != 0:
            input = torch.cat((input, input.new_zeros(input.shape[0], input.shape[1], input.shape[2],
                                                      input.shape[3] % kw, input.shape[4])), 3)
        n, c, h, w, t = input.shape
        result = conv_synapse(input.reshape(n, 1, c * h, w, t), self._weight(), self._stride2, self._padding2,
                              self._dilation2)
        return result.reshape(n, c, -1, result.shape[3], t)


class ConvTranspose(torch.nn.ConvTranspose3d, _SynapseLayer):
    """Transposed convolution synapse layer (synapse/layer.py:511-658 in the reference).

    Parameters
    ----------
    in_features, out_features : int
    kernel_size, stride, padding, dilation : int or (height, width)
    groups : int
    weight_scale, weight_norm, pre_hook_fx : as for :class:`Conv`.
    """

    def __init__(self, in_features, out_features, kernel_size, stride=1, padding=0, dilation=1, groups=1,
                 weight_scale=1, weight_norm=False, pre_hook_fx=None):
        kernel = _pair(kernel_size, 'kernel_size')
        self._stride2, self._padding2, self._dilation2 = _pair(stride, 'stride'), _pair(padding, 'padding'), \
            _pair(dilation, 'dilation')
        super().__init__(in_features, out_features, kernel + (1,), self._stride2 + (1,), self._padding2 + (0,), 0,
                         groups, False, self._dilation2 + (1,))
        self._finish(weight_scale, weight_norm, pre_hook_fx)

    def forward(self, input):
        """Weighted spikes [N, out_features, Ho, Wo, T] for spikes [N, in_features, H, W, T],
        Ho = (H - 1) stride - 2 padding + dilation (kh - 1) + 1."""
        return conv_transpose_synapse(input, self._weight(), self._stride2, self._padding2, self._dilation2,
                                      self.groups)


class Unpool(torch.nn.ConvTranspose3d, _SynapseLayer):
    """Unpooling synapse layer (synapse/layer.py:661-838 in the reference): every sample of a channel is spread
    over a window of ``kernel_size`` with a common weight (``weight_scale``, not trained).  As in the reference
    the channels are folded into the image height around a one-channel transposed convolution.

    Parameters
    ----------
    kernel_size, stride, padding, dilation : int or (height, width); ``stride`` defaults to ``kernel_size``.
    weight_scale, weight_norm, pre_hook_fx : as for :class:`Conv`.
    """

    def __init__(self, kernel_size, stride=None, padding=0, dilation=1, weight_scale=1, weight_norm=False,
                 pre_hook_fx=None):
        kernel = _pair(kernel_size, 'kernel_size')
        self._stride2 = kernel if stride is None else _pair(stride, 'stride')
        self._padding2, self._dilation2 = _pair(padding, 'padding'), _pair(dilation, 'dilation')
        super().__init__(1, 1, kernel + (1,), self._stride2 + (1,), self._padding2 + (0,), 0, 1, False,
                         self._dilation2 + (1,))
        self.weight = torch.nn.Parameter(weight_scale * torch.ones_like(self.weight), requires_grad=False)
        self._finish(1, weight_norm, pre_hook_fx)

    def forward(self, input):
        """Spread spikes [N, C, Ho, Wo, T] for spikes [N, C, H, W, T]."""
        n, c, h, w, t = input.shape
        result = conv_transpose_synapse(input.reshape(n, 1, c * h, w, t), self._weight(), self._stride2,
                                        self._padding2, self._dilation2)
        return result.reshape(n, c, -1, result.shape[3], t)

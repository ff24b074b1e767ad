"""Normalisations a neuron can apply between its synaptic input and its dynamics
(counterpart of neuron/norm.py in the reference: MeanOnlyBatchNorm :9-95, WgtScaleBatchNorm :98-230).

Plain torch modules, as in the reference: they run once per call on the [N, C, ..., T] tensor and are not part
of the time-sequential kernels.  A neuron that is given one of them hooks its weight quantiser into
``pre_hook_fx`` (neuron/base.py:127-141 in the reference)."""
import torch


def _identity(x, descale=False):
    return x


class _FeatureNorm(torch.nn.Module):
    """Per-feature (axis 1) running mean with momentum; the first input fixes the feature count."""

    def __init__(self, num_features, momentum, pre_hook_fx):
        super().__init__()
        self.num_features = num_features
        self.momentum = momentum
        self.pre_hook_fx = _identity if pre_hook_fx is None else pre_hook_fx
        self.register_buffer('running_mean', torch.zeros(1 if num_features is None else num_features))
        self.update = True

    @property
    def bias(self):
        """The mean as the (negative) bias a hardware neuron would carry."""
        return -self.pre_hook_fx(self.running_mean, descale=True)

    def _mean(self, inp):
        """Batch mean per feature while training (and updating), else the running estimate; also says
        whether the batch statistics were used."""
        if self.num_features is None:
            self.num_features = inp.shape[1]
        if self.training and self.update is True:
            mean = torch.mean(inp.reshape(inp.shape[0], self.num_features, -1), dim=[0, 2])
            with torch.no_grad():
                self.running_mean = (1 - self.momentum) * self.running_mean + self.momentum * mean
            return mean, True
        return self.running_mean, False

    @staticmethod
    def _per_feature(v, inp):
        if not 2 <= inp.dim() <= 5:
            raise AssertionError(f'Found unexpected number of dims {inp.dim()} in input.')
        return v.reshape((1, -1) + (1,) * (inp.dim() - 2))


class MeanOnlyBatchNorm(_FeatureNorm):
    """Subtracts the per-feature mean (batch mean while training, running mean otherwise); the
    subtracted value goes through ``pre_hook_fx`` first, so it can be quantised like a weight."""

    def __init__(self, num_features=None, momentum=0.1, pre_hook_fx=None):
        super().__init__(num_features, momentum, pre_hook_fx)

    def reset_parameters(self):
        self.running_mean.zero_()

    def forward(self, inp):
        mean, _ = self._mean(inp)
        return inp - self.pre_hook_fx(self._per_feature(mean, inp))


class WgtScaleBatchNorm(_FeatureNorm):
    """Mean subtraction plus a division by the standard deviation of the whole tensor rounded up to a power
    of two (exponent limited to +-``weight_exp_bits``), so that hardware can apply it as a shift."""

    def __init__(self, num_features=None, momentum=0.1, weight_exp_bits=3, eps=1e-5, pre_hook_fx=None):
        super().__init__(num_features, momentum, pre_hook_fx)
        self.weight_exp_bits = weight_exp_bits
        self.eps = eps
        self.register_buffer('running_var', torch.zeros(1))

    def reset_parameters(self):
        self.running_mean.zero_()
        self.running_var.zero_()

    def std(self, var):
        exponent = torch.ceil(torch.log2(torch.sqrt(var + self.eps)))
        return torch.pow(2., exponent.clamp(-self.weight_exp_bits, self.weight_exp_bits))

    @property
    def weight_exp(self):
        """Exponent of the equivalent weight scaling."""
        return torch.ceil(torch.log2(torch.sqrt(self.running_var + self.eps)))

    def forward(self, inp):
        mean, batch = self._mean(inp)
        if batch:
            var = torch.var(inp, unbiased=False)
            n = inp.numel() / inp.shape[1]
            with torch.no_grad():
                self.running_var = (1 - self.momentum) * self.running_var + self.momentum * var * n / (n + 1)
        else:
            var = self.running_var
        return (inp - self.pre_hook_fx(self._per_feature(mean, inp))) / self._per_feature(self.std(var), inp)

"""Neuron dropout (counterpart of neuron/dropout.py:10-35 in the reference)."""
import torch
import torch.nn.functional as F


class Dropout(torch.nn.Dropout3d):
    """Drops whole neurons: a dropped neuron stays silent for every time step of the sample (the surviving
    ones are scaled by 1 / (1 - p), as torch's dropout does)."""

    def forward(self, input):
        shape = input.shape
        per_neuron = input.reshape((shape[0], -1, 1, 1, shape[-1]))       # one channel per neuron, time last
        return F.dropout3d(per_neuron, self.p, self.training, self.inplace).reshape(shape)

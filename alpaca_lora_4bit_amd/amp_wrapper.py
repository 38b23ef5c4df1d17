"""Autocast wrapper with the interface of src/alpaca_lora_4bit/amp_wrapper.py:4-26
(`AMPWrapper(model, options).apply_forward()` / `.apply_generate()`).

Running the model under autocast is what makes `custom_fwd(cast_inputs=float16)` on the 4-bit
autograd Function cast activations and scales to fp16 before they reach the HIP kernels."""
import functools

import torch

_DEFAULT_OPTIONS = {'enabled': True, 'device_type': 'cuda'}


class AMPWrapper:
    """Rebinds `model.forward` / `model.generate` to versions that run inside
    `torch.amp.autocast(**options)`; the originals stay reachable as
    `model.non_autocast_forward` / `model.non_autocast_generate`."""

    def __init__(self, model, options=None):
        self.model = model
        self.options = dict(_DEFAULT_OPTIONS) if options is None else options

    def _wrap(self, method_name):
        saved_name = 'non_autocast_' + method_name
        setattr(self.model, saved_name, getattr(self.model, method_name))

        @functools.wraps(getattr(self.model, saved_name))
        def under_autocast(*args, **kwargs):
            with torch.amp.autocast(**self.options):
                return getattr(self.model, saved_name)(*args, **kwargs)

        setattr(self.model, method_name, under_autocast)
        return under_autocast

    def apply_forward(self):
        self.autocast_forward = self._wrap('forward')

    def apply_generate(self):
        self.autocast_generate = self._wrap('generate')

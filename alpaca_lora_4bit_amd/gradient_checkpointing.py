"""Activation checkpointing of the decoder blocks for LoRA finetuning, with the interface of the reference's
src/alpaca_lora_4bit/gradient_checkpointing.py:9-65 (`finetune.py:130-133` calls
`apply_gradient_checkpointing(model, checkpoint_ratio=...)`).

Every selected `LlamaDecoderLayer` gets its `forward` replaced by one that runs under
`torch.utils.checkpoint` while the layer is in training mode (`:17-31`; the original stays reachable as
`old_forward_for_cp`), and the first `nn.Embedding` returns a fresh leaf that requires grad (`:34-49`), so that
the checkpointed segments have a differentiable input although every base weight is frozen.  With a ratio
strictly between 0 and 1, `int(n * ratio)` blocks are picked evenly spaced from first to last (`:58-61`).
"""
import numpy as np
import torch
from torch.utils.checkpoint import checkpoint


def _decoder_layer_type():
    from transformers.models.llama.modeling_llama import LlamaDecoderLayer
    return LlamaDecoderLayer


class _ForwardPatch:
    """Replaces `target.forward` by `self.new_forward`; the original stays reachable as `old_forward_for_cp`
    (the attribute name the reference uses, gradient_checkpointing.py:18,41)."""

    def __init__(self, target):
        self._target = target
        self.apply_patch()

    def apply_patch(self):
        self._target.old_forward_for_cp = self._target.forward
        self._target.forward = self.new_forward

    def new_forward(self, *args, **kwargs):          # pragma: no cover - overridden
        raise NotImplementedError


class NewForward(_ForwardPatch):
    """Recompute-in-backward wrapper around one decoder block (`.layer`)."""

    @property
    def layer(self):
        return self._target

    def new_forward(self, *args, **kwargs):
        block = self._target
        if not block.training:
            return block.old_forward_for_cp(*args, **kwargs)
        # keyword arguments (masks, position embeddings, caches) ride in the closure, as in the reference
        return checkpoint(lambda *inputs: block.old_forward_for_cp(*inputs, **kwargs), *args, use_reentrant=True)


class VarWrapper(_ForwardPatch):
    """Cuts the graph after the embedding (`.model`): its output becomes a leaf that requires grad."""

    def __init__(self, model):
        super().__init__(model)
        print("Var Wrapper Patch Applied")

    @property
    def model(self):
        return self._target

    def new_forward(self, *args, **kwargs):
        return self._target.old_forward_for_cp(*args, **kwargs).detach().requires_grad_(True)


def checkpoint_locations(n_layers: int, checkpoint_ratio=1) -> np.ndarray:
    """Indices of the blocks that get checkpointed."""
    if 0 < checkpoint_ratio < 1:
        picks = np.linspace(0, 1, int(n_layers * checkpoint_ratio)) * (n_layers - 1)
        return np.array(picks.round(), dtype=int)
    return np.arange(n_layers)


def apply_gradient_checkpointing(model, checkpoint_ratio=1):
    """Patches `model` in place; returns (list of NewForward, VarWrapper of the first embedding or None)."""
    layer_type = _decoder_layer_type()
    blocks = [m for _, m in model.named_modules() if isinstance(m, layer_type)]
    patched = []
    for i in checkpoint_locations(len(blocks), checkpoint_ratio):
        patched.append(NewForward(blocks[i]))
        print("Forward Patch Applied For Block {}".format(i))
    wrapper = None
    for _, m in model.named_modules():
        if isinstance(m, torch.nn.Embedding):
            wrapper = VarWrapper(m)
            break
    return patched, wrapper

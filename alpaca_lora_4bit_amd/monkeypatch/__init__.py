"""Patches applied to third-party packages at run time (peft's LoRA model factory)."""

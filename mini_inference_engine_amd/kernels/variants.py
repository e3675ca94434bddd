"""Compile-time variants of the kernel modules that are built ahead of time.

attention_bf16 and prefill_attention_bf16 are built once per head size.  The sizes listed here are those of the
engine's benchmark shapes and tests; a model with another head size (any multiple of 16
up to 256) gets its variant compiled at first use.
"""

HEAD_DIMS = (16, 32, 48, 64, 80, 96, 128, 256)

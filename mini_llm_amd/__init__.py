"""A small, whole inference engine for GPT-2 on one MI355X: configuration and registry, weights,
parts and blocks, a paged cache, one step function, a scheduler and samplers, over hand-written
HIP kernels for gfx950."""

__version__ = "0.1.0"

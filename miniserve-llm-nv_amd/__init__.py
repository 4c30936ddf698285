"""A small, whole inference engine for one MI355X (gfx950): configuration,
weights, layers built from parts, a paged cache manager, one step function, a
scheduler, sampling, and hand-written HIP kernels underneath."""

__version__ = "0.1.0"

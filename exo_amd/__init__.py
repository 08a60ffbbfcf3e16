"""exo_amd: MI355X (gfx950) engine for exo's per-shard transformer forward on MLX
affine-quantised weights.  Compute runs in hand-written HIP kernels behind a C ABI
(include/exo_mi355x.h); this package is the Python host side."""

__version__ = "0.1.0"

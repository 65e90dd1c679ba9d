"""allpaca_amd: a single-GPU inference engine for MI355X (gfx950).

Layers, bottom to top: `csrc` (HIP kernels) and `kernels` (their loader and
checked wrappers); `parts` (mixer, feed-forward, norm, position encoding, block
arrangement); `models` (architectures that describe themselves with parts);
`weights`; `cache` (pages, block tables, state slots); `engine` (step function,
scheduler, requests); `sampling`; `cli`.
"""
__version__ = "0.1.0"

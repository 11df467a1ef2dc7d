"""holon_amd: a small, whole LLM inference engine for one AMD MI355X GPU, one architecture (Qwen3 dense), in the
shape of mxinO/holon: typed configuration and a registry, layers composed from parts, weights by tensor name, a paged
cache with block tables, one step function over mixed batches, a scheduler, sampling, and hand-written gfx950 HIP
kernels underneath."""

__version__ = "0.1.0"

"""qserve_amd -- MI355X (gfx950) implementation of QServe's W4A8KV4 hot path.

Layout:
  csrc/      hand-written HIP kernels + the C ABI (include/qserve_amd.h) -> libqserve_amd.so
  _lib.py    ctypes binding of that C ABI (no fallback: import fails loudly without the .so)
  backend/   host-side mirror of the reference's `qserve_backend.*` torch-extension modules
             (same callables / argument order / error behaviour); the top-level package
             `qserve_backend/` re-exports it under the reference's import names
  tp.py      tensor-parallel sharding of the packed weights + RCCL all-reduce
  decode.py  one Llama-style W4A8KV4 decode step expressed with the backend ops (bench / smoke driver)
  serving/   paged serving engine: model registry, paged cache + sequence slots, scheduler, sampler, command line, trace replay
  layers/    mechanisms the served models are made of (latent attention, rotary tables, mixture of experts) over an ops object
  models/    model definitions, registered by the architecture name of their config.json
  csrc/serve/  kernels of the serving engine -> libqserve_serve.so (include/qserve_serve.h), built on first use
"""
__version__ = "0.1.0"

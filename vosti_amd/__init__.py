"""vosti_amd: a small single-GPU inference engine for MI355X (gfx950).

Layers of the package, bottom up:

* ``csrc`` / ``kernels``: hand-written HIP kernels and their bindings
* ``config``: typed configurations and the architecture registry
* ``weights``: safetensors loading by tensor name, random-weights folders
* ``parts``: mixers, feed-forwards, norms, position encodings, blocks
* ``models``: a decoder assembled from parts as its configuration says
* ``cache``: paged-cache bookkeeping (native) and the tensors it indexes
* ``engine``: the step function, the scheduler and the generation loop
* ``sampling``: sampling parameters and per-request random state
"""
__version__ = "0.1.0"

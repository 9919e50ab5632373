"""levanter_amd: a one-GPU MI355X inference engine in the manner of marin-community/levanter.

Layout: ``config`` (typed configurations, the registry), ``weights`` (safetensors in and out,
random weights), ``parts`` (norms, position encodings, mixers, feed-forwards, blocks, the
decoder), ``models`` (architectures: configuration -> model description), ``cache`` (paged
keys and values, per-request state slots), ``engine`` (step function, scheduler, entry
point), ``sampling``, ``kernels`` (loader and launchers of the HIP library), ``csrc`` (HIP).
"""

__version__ = "0.1.0"

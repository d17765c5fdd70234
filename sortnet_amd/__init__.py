"""MI355X-native distance-neuron kernels for SortNet-style networks.

`sortnet_amd.norm_dist` (alias of `sortnet_amd.functional`) mirrors the functional/autograd API
of the reference's core/norm_dist.py; `sortnet_amd.ext` mirrors its compiled extension module;
both sit on libsortdist.so (hand-written HIP kernels for gfx950 behind a plain C ABI,
include/sortdist.h).  Submodules are imported explicitly, e.g.
`from sortnet_amd.norm_dist import norm_dist, sort_neuron`.
"""
__version__ = "0.1.0"

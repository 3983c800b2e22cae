"""MI355X (gfx950) kernels for the LSH bucket sort and the chunkwise gated-delta forward, behind the reference's names.

``lampa_amd.lsh`` (hashing, stable radix sort, gather / scatter), ``lampa_amd.hept`` (region front end of the HEPT
bucketing), ``lampa_amd.gated_delta`` (chunkwise and token-serial forward), ``lampa_amd.hgdn`` (hierarchical, level-weighted forward), ``lampa_amd.layer_ops`` (short convolution,
RMS norms, fused projection kernels), ``lampa_amd.block`` (a gated-delta layer and the 4-layer block). Everything runs
through ``liblampa_amd.so`` (``python -m lampa_amd.build``); there is no CPU fallback.
"""

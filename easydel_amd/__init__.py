"""MI355X-native ragged paged attention for EasyDeL's eSurge serving path.

``easydel_amd.operations`` mirrors the reference's operation registry and its ``ragged_page_attention_v2/_v3``
operations; ``easydel_amd.caching`` mirrors the paged KV cache they read; ``easydel_amd.kernels`` are the
tensor-level calls into ``librpa_hip.so`` (hand-written gfx950 kernels behind a C ABI, ``include/rpa_hip.h``).
"""

__version__ = "0.1.0"

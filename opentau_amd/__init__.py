"""MI355X-native block-causal (prefix-LM) attention: the one hot path of the
OpenTau-style VLA policies, as hand-written gfx950 kernels behind a C ABI.

``opentau_amd.flash_attn_hip`` mirrors the reference's op-level package
(``src/opentau/policies/flash_attn_cuda/__init__.py``); ``opentau_amd.attention``
mirrors the model-facing attention calls of the policies.
"""

__version__ = "0.1.0"

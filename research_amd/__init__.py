"""MI355X-native paged-KV attention for the `rollouts` inference engine.

Only the attention / KV-cache path lives here: the host-side mirror of the
reference interface in ``research_amd.inference`` and the HIP kernels behind a
C ABI in ``research_amd/csrc`` (built into ``libpaged_attn.so``).
"""

__version__ = "0.1.0"

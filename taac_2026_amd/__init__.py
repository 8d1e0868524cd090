"""taac_2026_amd - the unified pCVR token backbone's kernel path on MI355X (gfx950).

Hand-written HIP kernels (libtaac_hip.so, C ABI in include/taac_hip.h) behind the operator signatures of the
TAAC-2026 experiment workspace: ``rms_norm`` / ``layer_norm`` / ``flash_attention`` /
``scaled_dot_product_attention`` / ``RMSNorm`` / ``LayerNorm`` / ``SwiGLUFeedForward``. See ``taac_2026_amd.api``.
"""

__version__ = "0.1.0"

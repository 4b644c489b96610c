"""MI355X-native sparse shifted-window attention (operator set of SparseSwin3D).

``custom_ops``        the ten operators, same names/signatures as the reference's extension
``window_attention``  SparseTensor, autograd wrappers, WindowAttentionSparse
``layers``            SwinTransformerBlock, BasicLayer and the window index helpers
``synth``             seeded synthetic scenes (numpy only)

Importing the package does not load the HIP library; the first operator call does, and
raises if ``libsswin3d.so`` has not been built (``python -m sparseswin3d_amd.build``).
"""

__all__ = ["custom_ops", "window_attention", "layers", "synth"]

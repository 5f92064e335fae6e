"""MI355X-native F3M kernel-matrix-vector-product engine.

``f3m_amd.ffm_3d_float`` mirrors the reference's compiled module, ``f3m_amd.FFM_classes`` its
Python operator classes, ``f3m_amd.engine`` exposes plans (tree + interaction lists reused over
many right-hand sides).  Everything runs through the gfx950 library ``f3m_amd/lib/libf3m.so``.
"""
__all__ = ["engine", "ffm_3d_float", "FFM_classes", "capi"]

"""MI355X (gfx950) implementation of QMoE's compressed-expert inference path.

`qmoe_amd.sub1` mirrors the reference's `sub1.py` module surface (Sub1Linear,
setup, DEC/TRIE/DEV/GPUS); `qmoe_amd.sub1_hip` mirrors its `sub1_cuda`
extension (sub1matvec, sub1pack) on top of the C ABI in `include/sub1_hip.h`.
"""
__all__ = ['build', 'sub1', 'sub1_hip']

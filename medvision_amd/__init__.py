"""MI355X-native trilinear-sampling operators with MedVision's ``medvision.ops`` interface.

``medvision_amd.ops`` mirrors ``medvision/ops`` of the reference (RoIAlign, RoIAlignRotated,
DeformConv3d[Pack], ModulatedDeformConv3d[Pack], affine_*/apply_offset_* engines);
``medvision_amd._C`` mirrors the reference's pybind11 module on top of the C ABI of
``libmedvision_hip.so``.
"""
__version__ = "0.1.0"

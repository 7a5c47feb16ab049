"""MI355X-native fused normalization operators (fused RMSNorm, fused AdaLayerNorm)
behind the TeleTron `teletron_op` interface.  See teletron_amd.fusedlayers for the
autograd entry points and include/teletron_norm.h for the C ABI."""

__version__ = "0.1.0"

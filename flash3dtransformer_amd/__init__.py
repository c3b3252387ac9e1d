"""MI355X-native (gfx950) implementation of the Flash3D forward hot path.

Layout mirrors the reference package (`flash3dxfmr`):
  lib/     `pshattn` op surface over the C ABI of libf3d_hip.so
  psh/     buffer contracts, scope planning, batching helpers
  layers/  nn.Module API (Flash3D, Stage, XFMR, Hourglass, pooling, unpooling)
  csrc/    HIP kernels and the C ABI implementation
"""
__all__ = ["lib", "psh", "layers"]

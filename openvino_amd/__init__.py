"""MI355X-native FullyConnectedCompressed (weight-compressed FullyConnected) for OpenVINO.

The product is the C-ABI library ``libovfcc.so`` (HIP kernels for gfx950 + host repacker)
and the C++ OpenVINO plugin shim above it; this package is the Python host-side mirror used
by the tests and the benchmark.
"""
__version__ = "0.1.0"

"""MI355X-native int8 inference hot path (MatMul/FullConnection, Conv2D, DynamicQuant, dynamic MatMul) behind a
C-ABI shared library; this package is the Python host-side mirror used by tests and the benchmark."""

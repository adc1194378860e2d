"""nd4j-hip: an MI355X (gfx950) op backend for libnd4j's data-parallel op path.

csrc/            hand-written HIP kernels, host runtime and the C-ABI facade (libnd4jhip.so)
nativeops.py     ctypes binding of the C ABI (stand-in for the JavaCPP-generated binding class)
ndarray.py       host-side array handle (stand-in for INDArray / OpaqueNDArray)
executioner.py   op executioner following the Java NativeOpExecutioner's call protocol
"""

"""Python faces of the three reference extension modules (minimax, quantization, calc_precision).

Each module keeps the reference's function names, argument order and error behaviour and forwards to
libgact_hip.so through its C ABI (see _abi.py).
"""

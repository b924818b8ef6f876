"""MI355X-native quantized-KV decode attention (the hot path of HqeKV) behind the reference's
operator interface: hand-written HIP kernels for gfx950 in ``libhqekv.so`` (C ABI, ``include/hqekv.h``)
and thin Python modules that keep the reference's function names and the 42-field cache tuple."""
__all__ = ["pack_unpack", "matmul", "quant_matmul_hq", "hqe_matmul", "hybrid_quant", "hqe_2",
           "public_func", "attention", "cache_policy", "synth", "compat"]
__version__ = "0.1.0"

"""MI355X-native implementation of ADKV's streaming EMA delta quantizer and decode attention.

Layout:
  csrc/          hand-written HIP kernels for gfx950 and the C ABI (include/adkv_hip.h)
  build.py       hipcc driver that produces libadkv_hip.so next to this file
  _lib.py        ctypes loader; raises if the library is missing (there is no CPU fallback)
  kernel/gemv.py drop-in for the reference's adkv.kernel.gemv (encode_kv, forward_qk, forward_ov)
  hf/            host-side cache object mirroring the reference's Hugging Face integration
"""

__version__ = "0.1.0"

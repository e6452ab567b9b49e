"""MI355X-native KV-cache hot path of warp34: TQ4 quantize-on-append into paged KV blocks and
paged GQA decode / verify attention, behind the reference's C ABI (include/warp34_kv.h)."""
from . import ffi  # noqa: F401
from .ffi import load  # noqa: F401

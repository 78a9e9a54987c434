"""One file holding a whole quantized model (llmquant/packing)."""

from llmquant.packing.format import read_header, read_packed, write_packed
from llmquant.packing.packing import pack_int4, pack_weight, unpack_int4, unpack_weight

__all__ = ["pack_int4", "pack_weight", "read_header", "read_packed", "unpack_int4",
           "unpack_weight", "write_packed"]

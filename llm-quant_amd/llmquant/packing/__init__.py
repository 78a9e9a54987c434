"""One file holding a whole quantized model (llmquant/packing)."""

from llmquant.packing.format import read_header, read_packed, write_packed
from llmquant.packing.packing import pack_int4, pack_weight, unpack_int4, unpack_weight

__all__ = ["describe_packed", "load_packed_model", "pack_int4", "pack_weight", "packed_dtypes", "read_header",
           "read_packed", "save_packed_model", "unpack_int4", "unpack_weight", "write_packed"]

_MODEL_IO = ("describe_packed", "load_packed_model", "packed_dtypes", "save_packed_model")


def __getattr__(name):
    # model_io needs the kernel-mode module class; imported on first use so that the byte-level
    # helpers above stay importable from llmquant.quantizers.kernel without a cycle
    if name in _MODEL_IO:
        from llmquant.packing import model_io

        return getattr(model_io, name)
    raise AttributeError(name)

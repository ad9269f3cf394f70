"""`Metadata(dim)` factory (reference: sparseconvnet/metadata.py:14-17)."""
from . import SCN


def Metadata(dim):
    if dim != 3:
        raise NotImplementedError("only 3-d sparse tensors are provided")
    return SCN.Metadata_3()

"""Import-path compatibility: the reference exposes its quantizers as src.quantizers.*."""
from hqmq_amd.quantizer import (KVQuantizer, HQMQQuantizer, OutlierAwareHQMQQuantizer, OutlierAwareGenericQuantizer,
                                PaddedHQMQQuantizer)

__all__ = ["KVQuantizer", "HQMQQuantizer", "OutlierAwareHQMQQuantizer", "OutlierAwareGenericQuantizer",
           "PaddedHQMQQuantizer"]

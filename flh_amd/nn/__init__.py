from .linear import LinearFLH  # noqa: F401
from .normalization import RMSNorm  # noqa: F401
from .quantization import Quantizer, ActQuantizer, WeightQuantizer, fast_hadamard_transform  # noqa: F401
from .hadamard import OnlineHadamard  # noqa: F401
from . import linear_gs, quantization_gs  # noqa: F401
from .fused import RMSNormQuant, SiluMulQuant  # noqa: F401
from .checkpoint import save_quantized, load_quantized  # noqa: F401
from .gptq import FLHGPTQ, GPTQQuantizer  # noqa: F401

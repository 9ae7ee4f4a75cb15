"""jitnn_amd: MI355X (gfx950) implementation of jitNN's GGUF quantised-weight linear path.

The arithmetic lives in libjitnn_hip.so (C ABI: include/jitnn_hip.h); this package is the thin host
mirror of the reference's Tensor / Gguf / Quant / F interface for that path, used by the tests and the
benchmark.  Importing it requires the built library.
"""
from ._lib import JitnnError, device_info, init, stats, stats_reset  # noqa: F401
from .dtype import DType  # noqa: F401
from .ops import F, Gguf, Quant  # noqa: F401
from .tensor import Tensor  # noqa: F401
from .llama import LlamaDecoder  # noqa: F401
from .gguf_file import GgufFile, GgufTensorInfo  # noqa: F401
from ._lib import UnsupportedTypeError  # noqa: F401
from .tokenizer import Tokenizer  # noqa: F401
from .llm import GenerationRequest, GenerationResult, Llm, ModelInfo  # noqa: F401

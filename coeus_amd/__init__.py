"""coeus_amd: the transformer forward pass of rustllm-core's model-transformer plugin on one
MI355X (gfx950), behind the reference's plugin surface.  Kernels and the C ABI live in
csrc/ (built into libcoeus_mi355x.so); plugin.py mirrors the reference's host interface."""
from .plugin import (BasicGenerationConfig, ConfigError, CoeusError, DeviceError, ProcessingError, Session,  # noqa: F401
                     Transformer250MConfig, TransformerModel, TransformerModelBuilder,
                     TransformerModelPlugin)
from .serialization import read_rustllm, write_rustllm  # noqa: F401,E402
from .tokenizer import BpeTokenizer, BpeTokenizerPlugin, StringToken  # noqa: F401,E402

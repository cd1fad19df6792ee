"""wgml_amd — MI355X (gfx950) batch-1 token-decode path behind wgml's operator API.

Everything computes in `lib/libwgml_hip.so` (hand-written HIP kernels behind a C
ABI, see include/wgml_hip.h); this package is the thin host-side mirror of the
reference's `wgml::ops` / `wgml::models` names.  Importing fails if the library
has not been built: there is no CPU fallback.
"""
from ._lib import (F16, F32, Q4_0, Q4_1, Q4_K, Q5_0, Q5_1, Q5_K, Q6_K, Q8_0, Q8_K, LIB_PATH,  # noqa: F401
                   WgmlError, lib)
from .ops import *  # noqa: F401,F403
from .models import *  # noqa: F401,F403
from .models import prompt_tokens  # noqa: F401
from .gguf import (Gguf, GgufTensor, gpt2_params_from_gguf, gpt2_weights_from_gguf,  # noqa: F401
                   llama2_config_from_gguf, llama2_weights_from_gguf)
from .tokenizer import Gpt2Tokenizer, LlamaTokenizer, llama2_chat_prompt  # noqa: F401
from .chat_template import ChatTemplate, Prompt, TemplateError, LLAMA2_CHAT_TEMPLATE  # noqa: F401

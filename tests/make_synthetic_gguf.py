"""The GGUF writer lives in the package (llama.cpp_amd/mi355/gguf.py); tests keep importing it under this name."""
from mi355.gguf import *          # noqa: F401,F403
from mi355.gguf import write_model, tensor_list, use_more_bits   # noqa: F401

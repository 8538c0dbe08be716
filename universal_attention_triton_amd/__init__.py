"""Universal Attention for AMD Instinct MI355X: hand-written HIP kernels (libua_hip.so) behind the
Python interface of spikerheado1234/Universal_Attention_triton."""
from .universal_attention import UniversalAttention, attention, universal_attention  # noqa: F401
from .universal_attention_autograd import SMVecMatMul, UniversalAttention2  # noqa: F401
from .universal_attention_autograd import UniversalAttention as UniversalAttention1D  # noqa: F401

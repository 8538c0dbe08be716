"""Drop-in module path of the reference (`from universal_attention_autograd import UniversalAttention, ...`);
the implementation lives in universal_attention_triton_amd."""
from universal_attention_triton_amd.universal_attention_autograd import SMVecMatMul, UniversalAttention, UniversalAttention2  # noqa: F401

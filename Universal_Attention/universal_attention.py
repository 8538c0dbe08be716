"""Drop-in module path of the reference (`from Universal_Attention.universal_attention import UniversalAttention`);
the implementation lives in universal_attention_triton_amd."""
from universal_attention_triton_amd.universal_attention import UniversalAttention, attention, universal_attention  # noqa: F401

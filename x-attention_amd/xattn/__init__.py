"""MI355X-native XAttention prefill operator.

Import path and public names follow mit-han-lab/x-attention
(``from xattn.src.Xattention import Xattention_prefill, xattn_estimate``) so
that model integrations written against it import unchanged.
"""

"""nanoplm_amd: MI355X-native varlen depthwise 1-D convolution for nanoPLM's packed conv path."""
from .dwconv import (  # noqa: F401
    VarlenDWConv1d,
    VarlenDWConv1dFunction,
    bwd_workspace_bytes,
    check_cu_seqlens,
    varlen_dwconv,
    varlen_dwconv_bwd,
    varlen_dwconv_bwd_op,
    varlen_dwconv_compilable,
    varlen_dwconv_fwd,
    varlen_dwconv_fwd_op,
)
from .padded import (  # noqa: F401
    is_right_padded,
    pad_output,
    padded_dwconv,
    right_padded_cu_seqlens,
    unpad_input,
)
from .gated import (  # noqa: F401
    GatedVarlenDWConv1dFunction,
    gated_dwconv_bwd,
    gated_dwconv_bwd_op,
    gated_dwconv_fwd,
    gated_dwconv_fwd_op,
    gated_supported,
    gated_varlen_dwconv,
)
from .lnconv import (  # noqa: F401
    LnVarlenDWConv1dFunction,
    ln_dwconv_bwd,
    ln_dwconv_bwd_op,
    ln_dwconv_fwd,
    ln_dwconv_fwd_op,
    ln_supported,
    ln_varlen_dwconv,
    ln_varlen_dwconv_compilable,
)
from .hygiene import conv_parameters, split_conv_parameters  # noqa: F401

__version__ = "0.1.0"

"""Fused entropy-decode + GEMV for losslessly compressed BF16 weights on MI355X.

Drop-in for the Python surface of lszxb/bf16_huffman_infer::

    import bf16_huffman_infer_amd as bf16_huffman_infer
    bf16_huffman_infer.convert_all_linear(model, min_out_features=0, algo='huffman')
"""
from .functional import *  # noqa: F401,F403
from .functional import mv_ans, mv_huffman  # noqa: F401
from .utils import get_model_size  # noqa: F401
from .cudagraph_utils import get_graphed_model  # noqa: F401,E402

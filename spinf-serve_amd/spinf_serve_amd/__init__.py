"""MI355X-native tree-mask packed-prefill attention and Gated DeltaNet scan behind the reference's call boundary.

  layout      TokenTree / Batch / pack_stream: the stream layout of packed token trees (spinf_serve/packer.py:352-423)
  masks       TreeMask, block_masks: the mask side of the boundary (spinf_serve/scorer.py:163-238)
  attention   tree_attn custom op, tree_flex_forward, tree_attention (gemma4.py:98-119, qwen.py:604-623)
  gdn         recurrent, chunked (spinf_serve/models/qwen35/gdn.py)
  qwen_plan   tree_plan, gdn_tree (spinf_serve/models/qwen35/qwen.py:158-276, 514-590)
  decode      XCaches, GroupKV, x_attention: the extraction decoder's attention step (spinf_serve/decode.py:35-104)
  synth       seeded synthetic workloads of the benchmark configurations

All device work goes through libspinf_tree.so (HIP, gfx950); there is no CPU or PyTorch fallback: importing the
compute entry points without the built library raises.
"""

from ._lib import load_library, library_path  # noqa: F401
from .layout import BLOCK, Batch, TokenTree, pack_stream, pack_streams  # noqa: F401
from .masks import TreeMask, TilePlan, block_masks  # noqa: F401
from .attention import CAPTURE, register_tree_attention, tree_attention, tree_attn, tree_attn_noalloc, tree_flex_forward  # noqa: F401
from .gdn import chunked, recurrent  # noqa: F401
from .gdn_layer import gdn_gate, gdn_prologue  # noqa: F401
from .lm_head import lm_head_logprobs, lm_logprobs  # noqa: F401
from .decode import GroupKV, XCaches, x_attention, xdecode_attn  # noqa: F401
from .qwen_plan import Call, TreePlan, gdn_tree, tree_plan  # noqa: F401

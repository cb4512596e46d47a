"""ComfyUI custom-node package: installs risaattention_amd's attention into a MODEL.

Link this directory (not the repository root) into ``ComfyUI/custom_nodes``; the
attention library itself stays importable as ``risaattention_amd``.
"""

from .node import RISAAttentionNode

NODE_CLASS_MAPPINGS = {"RISAAttention": RISAAttentionNode}
NODE_DISPLAY_NAME_MAPPINGS = {"RISAAttention": "RISA Attention"}

__all__ = ["NODE_CLASS_MAPPINGS", "NODE_DISPLAY_NAME_MAPPINGS"]

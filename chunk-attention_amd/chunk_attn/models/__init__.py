"""Host-side callers of the decode path: request objects, the iteration-level scheduler and a
small attention-only language model to drive them (mirrors src/chunk_attn/models of the
reference project)."""
from .sequence import Sequence  # noqa: F401
from .model_host import ModelHost  # noqa: F401

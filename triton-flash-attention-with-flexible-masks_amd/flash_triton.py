"""Drop-in module name: code that does ``from flash_triton import attention`` keeps
working when this directory precedes the reference on ``sys.path``.  It only
re-exports the gfx950 operator; nothing in here uses Triton."""
from flash_mi355 import (SCORE_FUNC_MODE0_NOPE, SCORE_FUNC_MODE1_DOC, FlashAttention,  # noqa: F401
                         attention, maybe_contiguous)

"""Type aliases (reference: flash_dropout/types.py:1-3)."""
import torch.types

size = torch.types._size

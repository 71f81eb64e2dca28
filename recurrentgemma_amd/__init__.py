"""MI355X-native Conv1D + RG-LRU recurrent-block core (drop-in for the
`recurrentgemma.torch` modules of the same names)."""

from recurrentgemma_amd.layers import BlockDiagonalLinear
from recurrentgemma_amd.layers import Conv1D
from recurrentgemma_amd.layers import RGLRU
from recurrentgemma_amd.layers import rnn_param_init
from recurrentgemma_amd.layers import rnn_scan
from recurrentgemma_amd.modules import RecurrentBlock
from recurrentgemma_amd.modules import RecurrentBlockCache
from recurrentgemma_amd.modules import recurrent_core

__all__ = [
    "BlockDiagonalLinear", "Conv1D", "RGLRU", "RecurrentBlock",
    "RecurrentBlockCache", "recurrent_core", "rnn_param_init", "rnn_scan",
]

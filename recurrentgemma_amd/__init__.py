"""MI355X-native Conv1D + RG-LRU recurrent-block core (drop-in for the
`recurrentgemma.torch` modules of the same names), and the residual stack and
sampler that call it."""

from recurrentgemma_amd import training
from recurrentgemma_amd.layers import BlockDiagonalLinear
from recurrentgemma_amd.layers import Conv1D
from recurrentgemma_amd.layers import RGLRU
from recurrentgemma_amd.layers import rnn_param_init
from recurrentgemma_amd.layers import rnn_scan
from recurrentgemma_amd.griffin import AttentionBlockCache
from recurrentgemma_amd.griffin import Embedder
from recurrentgemma_amd.griffin import Griffin
from recurrentgemma_amd.griffin import GriffinConfig
from recurrentgemma_amd.griffin import LocalAttentionBlock
from recurrentgemma_amd.griffin import MLPBlock
from recurrentgemma_amd.griffin import Preset
from recurrentgemma_amd.griffin import ResidualBlock
from recurrentgemma_amd.griffin import RMSNorm
from recurrentgemma_amd.griffin import TemporalBlockType
from recurrentgemma_amd.modules import RecurrentBlock
from recurrentgemma_amd.modules import RecurrentBlockCache
from recurrentgemma_amd.modules import recurrent_core
from recurrentgemma_amd.sampler import Sampler
from recurrentgemma_amd.sampler import SamplerOutput

__all__ = [
    "AttentionBlockCache", "BlockDiagonalLinear", "Conv1D", "Embedder",
    "Griffin", "GriffinConfig", "LocalAttentionBlock", "MLPBlock", "Preset",
    "RGLRU", "RMSNorm", "RecurrentBlock", "RecurrentBlockCache",
    "ResidualBlock", "Sampler", "SamplerOutput", "TemporalBlockType",
    "recurrent_core", "rnn_param_init", "rnn_scan", "training",
]

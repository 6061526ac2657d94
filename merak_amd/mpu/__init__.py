"""Model parallel utility interface (the names Merak/core/mpu/__init__.py:22-56 exports for this path)."""

from .cross_entropy import vocab_parallel_cross_entropy
from .cross_entropy import vocab_parallel_cross_entropy_partials
from .cross_entropy import vocab_parallel_cross_entropy_backward_
from .cross_entropy import vocab_loss_fn
from .cross_entropy import lm_head_cross_entropy

from .initialize import destroy_model_parallel
from .initialize import get_model_parallel_group, set_model_parallel_group
from .initialize import get_model_parallel_rank, set_model_parallel_rank
from .initialize import get_model_parallel_world_size, set_model_parallel_world_size

from .layers import ColumnParallelLinear
from .layers import RowParallelLinear
from .layers import VocabParallelEmbedding

from .mappings import copy_to_model_parallel_region
from .mappings import gather_from_model_parallel_region
from .mappings import reduce_from_model_parallel_region
from .mappings import scatter_to_model_parallel_region

from .random import get_rng_tracker
from .random import model_parallel_manual_seed
from .random import RNGStatesTracker

from .utils import divide
from .utils import ensure_divisibility
from .utils import split_tensor_along_last_dim
from .utils import VocabUtility

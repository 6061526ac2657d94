from .mp_layers import ColPara, RowPara, build_layers
from .utils import init_method_normal, scaled_init_method_normal

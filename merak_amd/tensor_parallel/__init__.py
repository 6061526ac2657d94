from .mp_layers import ColPara, RowPara, build_layers
from .mp_attrs import (set_tp_layer_lists, set_mp_attr, rebuild_module, mp_is_setted, get_tp_attr_list,
                       reset_tp_layer_lists)
from .utils import init_method_normal, scaled_init_method_normal

from .compiler import CuteInductor
from .rmsnorm import replace_rmsnorm
from .swiglu_unchunked import replace_swiglu_unchunked

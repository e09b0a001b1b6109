from .contiguous import ensure_contiguous, ensure_same_strides
from .custom_op import cute_op, set_cute_tracing
from .device import device_synchronize, get_cu_count, get_sm_count
from .env import get_boolean_env_variable

from .cache import get_cutotune_cache, save_cutotune_cache
from .config import CutoTuneConfig, get_cartesian_product_cutotune_configs
from .parameter import CutoTuneParameter
from .tuner import cutotune

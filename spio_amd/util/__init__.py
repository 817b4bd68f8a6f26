"""Small host-side helpers shared by the conv2d_gw8 path."""

from .math import divup, next_relative_prime
from .close import assert_all_close, assert_all_close_with_acc_depth
from .tensor_format import to_channels_last
from .memory_format import check_channels_last
from .env import env_var_is_true
from .logger import logger_enabled, logger_verbose, log_level
from .interval_timer import Timer, time_function
from .device_info import get_device_ordinal, get_formatted_device_name, get_formatted_arch
from .cache_dir import get_cache_dir

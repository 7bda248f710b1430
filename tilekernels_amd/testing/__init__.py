from .generator import (generate_hidden_sizes, generate_moe_layout, generate_num_tokens,  # noqa: F401
                        make_baseline_input)
from .numeric import assert_equal, calc_diff, check_bias, count_bytes  # noqa: F401
from .quant import clear_unused_sf  # noqa: F401

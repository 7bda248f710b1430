from .bench import dtype_to_str, make_param_id, make_param_key  # noqa: F401
from .generator import (generate_e5m6_inputs, generate_hidden_sizes, generate_moe_layout, generate_moe_params,  # noqa: F401
                        generate_num_sms, generate_num_tokens, generate_rand_float, generate_topk_idx, make_baseline_input)
from .numeric import assert_equal, calc_diff, check_bias, count_bytes  # noqa: F401
from .quant import clear_unused_sf  # noqa: F401

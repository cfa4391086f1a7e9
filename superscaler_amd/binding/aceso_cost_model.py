"""The reference-side binding: copy this file to the reference's search/aceso_cost_model.py (keep the original
beside it as aceso_cost_model_cpu.py).  aceso_search.py, aceso_prims.py, aceso_policy.py and gen_megatron_plan.py
then run unchanged on the MI355X evaluator: the names they import (search/aceso_search.py:4, aceso_prims.py:7,
gen_megatron_plan.py:8) come from superscaler_amd.aceso_cost_model, with the reference's signatures.

It is the only file of this package that imports the reference's own modules (aceso_utils for the argparse
singleton), so it lives outside the package's import path and is never imported by the package itself."""
from aceso_utils import parse_args                 # the reference's flag system (search/aceso_utils.py:455-531)

import superscaler_amd.aceso_cost_model as _gpu

args = parse_args()                                # the import-time singleton of search/aceso_cost_model.py:10
_gpu.configure(args)                               # hands the namespace over; no GPU work before the first scoring call

from superscaler_amd.aceso_cost_model import (     # noqa: E402  same names, same signatures
    read_profiled_time, predict_time_breakdown, predict_stage_time, predict_stage_memory,
    predict_value_after_move, wrap_predict_delta_time, predict_stage_time_helper,
    predict_stage_memory_helper, check_recompute, update_recompute, get_reserved_memory_list,
    get_activation_size,
    predict_time_breakdown_batch)                  # + the batched entry point (one launch for a list of plans)

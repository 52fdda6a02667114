"""One-rank stand-in for the reference's `llm.utils.env.dist_env` (Megatron "mpu").

At TP = PP = DP = 1 every mapping of the reference is the identity
(llm/utils/env/dist_env/dist_mappings.py:52-53,67-68,86-87,108-109,130-131,148-149) and its
parameter AVG all-reduces (fused_layer_norm.py:51-54, row_parallel_linear.py:121-124) act on a
one-rank group.  This module keeps the call shape the layers use and nothing else; collectives
across GPUs are outside this build.
"""
import contextlib


def get_tensor_model_parallel_world_size():
    return 1


def get_tensor_model_parallel_rank():
    return 0


def get_pipeline_model_parallel_world_size():
    return 1


def get_pipeline_model_parallel_rank():
    return 0


def get_data_parallel_world_size():
    return 1


def get_data_parallel_rank():
    return 0


def get_tensor_model_parallel_group():
    return None


def is_pipeline_first_stage():
    return True


def is_pipeline_last_stage():
    return True


def copy_to_tensor_model_parallel_region(x):
    return x


def reduce_from_tensor_model_parallel_region(x):
    return x


def scatter_to_tensor_model_parallel_region(x):
    return x


def gather_from_tensor_model_parallel_region(x):
    return x


def scatter_to_sequence_parallel_region(x):
    return x


def gather_from_sequence_parallel_region(x, tensor_parallel_output_grad=True):
    return x


def reduce_scatter_to_sequence_parallel_region(x):
    return x


def sync_tp_duplicated_parameter(param):
    """AVG all-reduce over a one-rank group: nothing to do."""
    return param


class _RngTracker(object):
    """`get_cuda_rng_tracker().fork()` guards dropout in the reference (transformer.py:489); with
    dropout 0 and one rank there is no state to switch."""

    @contextlib.contextmanager
    def fork(self, name="model-parallel-rng"):
        yield


_TRACKER = _RngTracker()


def get_cuda_rng_tracker():
    return _TRACKER

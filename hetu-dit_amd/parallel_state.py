"""One-GPU stand-ins for the reference's parallel-state getters
(``hetu_dit/core/distributed/parallel_state.py:69-216``).  Every world size is
1 and every rank 0, so each collective on the hot path is bypassed exactly as
the reference bypasses it at world size 1
(``group_coordinator.py:219-220,:231-233``)."""


class _SingleRankGroup:
    """What ``get_tp_group()`` hands back at one GPU: collectives are no-ops."""

    world_size = 1
    rank_in_group = 0

    def all_reduce(self, tensor):
        return tensor

    def all_gather(self, tensor, dim=0, separate_tensors=False):
        return [tensor] if separate_tensors else tensor


_GROUP = _SingleRankGroup()


def get_tensor_model_parallel_world_size() -> int:
    return 1


def get_tensor_model_parallel_rank() -> int:
    return 0


def get_sequence_parallel_world_size() -> int:
    return 1


def get_sequence_parallel_rank() -> int:
    return 0


def get_ulysses_parallel_world_size() -> int:
    return 1


def get_ring_parallel_world_size() -> int:
    return 1


def get_pipeline_parallel_world_size() -> int:
    return 1


def get_pipeline_parallel_rank() -> int:
    return 0


def get_classifier_free_guidance_world_size() -> int:
    return 1


def get_data_parallel_world_size() -> int:
    return 1


def is_pipeline_first_stage() -> bool:
    return True


def is_pipeline_last_stage() -> bool:
    return True


def get_tp_group() -> _SingleRankGroup:
    return _GROUP

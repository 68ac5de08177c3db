"""Builds buffers from the reference's `replay_buffer` config entry.

Mirrors MSRL.__create_replay_buffer (mindspore_rl/core/msrl.py:270-300): the entry
names the class under 'type', an optional 'number' of instances, either a 'params'
dict or 'sample_size' / 'capacity', and the per-element 'data_shape' / 'data_type'
that the algorithm's session fills in (mindspore_rl/algorithm/dqn/dqn_session.py:50-61).
"""


def create_replay_buffer(replay_buffer_config):
    """Returns one buffer, or a list of `number` buffers, for a config dict such as
    {'number': 1, 'type': UniformReplayBuffer, 'capacity': 100000, 'sample_size': 64,
     'data_shape': [(4,), (1,), (1,), (4,)], 'data_type': [float32, int32, float32, float32]}."""
    num_replay_buffer = replay_buffer_config.get("number", 1)
    replay_buffer_type = replay_buffer_config["type"]
    params = replay_buffer_config.get("params", None)
    if not params:
        params = {
            "sample_size": replay_buffer_config.get("sample_size", 1),
            "capacity": replay_buffer_config.get("capacity"),
        }
    else:
        params = dict(params)
    params["shapes"] = tuple(replay_buffer_config.get("data_shape"))
    params["types"] = tuple(replay_buffer_config.get("data_type"))
    if num_replay_buffer == 1:
        return replay_buffer_type(**params)
    return [replay_buffer_type(**params) for _ in range(num_replay_buffer)]

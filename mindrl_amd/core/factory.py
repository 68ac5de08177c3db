"""Builds buffers from the `replay_buffer` entry of a MindRL algorithm config.

The entry's schema is the reference's (mindspore_rl/core/msrl.py:270-300, filled in by the
algorithm's session, e.g. mindspore_rl/algorithm/dqn/dqn_session.py:50-61):

    type         the buffer class (required)
    number       how many instances to build (default 1; more than one returns a list)
    params       constructor keywords, OR
    sample_size  (default 1) and
    capacity     when there is no `params`
    data_shape   per-field shapes  -> constructor keyword `shapes`
    data_type    per-field dtypes  -> constructor keyword `types`
"""

_KNOWN_KEYS = frozenset(["type", "number", "params", "sample_size", "capacity", "data_shape", "data_type"])


class ReplayBufferSpec:
    """A validated `replay_buffer` config entry: which class to build, how often, with which keywords."""

    def __init__(self, entry):
        if not isinstance(entry, dict):
            raise TypeError("a replay_buffer config entry is a dict, got %s" % type(entry).__name__)
        unknown = sorted(set(entry) - _KNOWN_KEYS)
        if unknown:
            raise KeyError("unknown replay_buffer config keys: %s" % ", ".join(map(str, unknown)))
        if "type" not in entry:
            raise KeyError("the replay_buffer config entry names no 'type'")
        if entry.get("data_shape") is None or entry.get("data_type") is None:
            raise KeyError("the replay_buffer config entry needs 'data_shape' and 'data_type'")
        self.cls = entry["type"]
        self.count = int(entry.get("number", 1))
        if self.count < 1:
            raise ValueError("'number' must be at least 1, got %d" % self.count)
        explicit = entry.get("params")
        if explicit:
            self.kwargs = dict(explicit)  # a copy: the caller's config is left as it is
        else:
            self.kwargs = {"sample_size": entry.get("sample_size", 1), "capacity": entry.get("capacity")}
        self.kwargs.update(shapes=tuple(entry["data_shape"]), types=tuple(entry["data_type"]))

    def build(self):
        made = [self.cls(**self.kwargs) for _ in range(self.count)]
        return made[0] if self.count == 1 else made


def create_replay_buffer(replay_buffer_config):
    """One buffer, or a list of `number` buffers, for an entry such as
    {'number': 1, 'type': UniformReplayBuffer, 'capacity': 100000, 'sample_size': 64,
     'data_shape': [(4,), (1,), (1,), (4,)], 'data_type': [float32, int32, float32, float32]}."""
    return ReplayBufferSpec(replay_buffer_config).build()


class ReplayBufferSet:
    """The buffers of the `replay_buffer` section of an algorithm config, as MSRL holds them
    (mindspore_rl/core/msrl.py:407-421):

    * a plain entry builds `buffers` (one buffer, or a list when `number` > 1); for a single buffer its
      sample / insert / full / reset are bound as `replay_buffer_sample`, `replay_buffer_insert`,
      `replay_buffer_full`, `replay_buffer_reset`, the names the trainers call
      (mindspore_rl/algorithm/dqn/dqn_trainer.py:80,83);
    * a section with a true `multi_type_replaybuffer` holds one entry per name; `buffers` is then a dict
      name -> buffer(s) and nothing is bound.
    """

    _HANDLERS = ("sample", "insert", "full", "reset")

    def __init__(self, section):
        if not isinstance(section, dict):
            raise TypeError("the replay_buffer section is a dict, got %s" % type(section).__name__)
        if section.get("multi_type_replaybuffer"):
            self.buffers = {name: create_replay_buffer(entry) for name, entry in section.items()
                            if name != "multi_type_replaybuffer"}
            return
        entry = {k: v for k, v in section.items() if k != "multi_type_replaybuffer"}
        self.buffers = create_replay_buffer(entry)
        if not isinstance(self.buffers, list):
            for name in self._HANDLERS:
                setattr(self, "replay_buffer_" + name, getattr(self.buffers, name))

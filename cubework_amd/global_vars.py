"""Process-wide tensor-parallel settings the layer constructors read.

The interface of cubework/global_vars.py:30-80 of the reference: `env.mode`
selects the 1d/2d/3d implementation, `env.parallel_input_1d` and
`env.vocab_parallel` are side channels that constructors toggle, and the 3D
group names are swapped after every Linear3D. `env.load(**settings)` replaces
every setting (unnamed ones return to their defaults), `env.save()` returns
them as a dict that `load` takes back.
"""
ALLOWED_MODES = (None, "1d", "2d", "3d")

# attribute that parameters carry: the number of ranks a parameter is split over
NUM_PARTITIONS = "NUM_PARTITIONS"

# names of the five process groups of the 3D layout
PARALLEL_3D_INPUT, PARALLEL_3D_WEIGHT, PARALLEL_3D_OUTPUT = ("PARALLEL_3D_" + n for n in ("INPUT", "WEIGHT", "OUTPUT"))
PARALLEL_3D_INPUT_X_WEIGHT = PARALLEL_3D_INPUT + "_X_WEIGHT"
PARALLEL_3D_OUTPUT_X_WEIGHT = PARALLEL_3D_OUTPUT + "_X_WEIGHT"

# setting -> default
_DEFAULTS = {
    "mode": None,
    "vocab_parallel": False,
    "parallel_input_1d": False,
    "summa_dim": None,
    "depth_3d": None,
    "input_group_3d": None,
    "weight_group_3d": None,
    "output_group_3d": None,
    "input_x_weight_group_3d": None,
    "output_x_weight_group_3d": None,
}


class TensorParallelEnv:
    """The one settings object of the process (`env` below); every setting is a plain attribute."""

    def __init__(self, **settings):
        self.load(**settings)

    def load(self, **settings):
        unknown = set(settings) - set(_DEFAULTS)
        if unknown:
            raise TypeError("unknown tensor-parallel settings: %s" % ", ".join(sorted(unknown)))
        for name, default in _DEFAULTS.items():
            setattr(self, name, settings.get(name, default))

    def save(self):
        return {name: getattr(self, name) for name in _DEFAULTS}


env = TensorParallelEnv()

"""Global, typed configuration bag (reference: mobula/config.py:4-66).

Only the keys that matter on this path are kept; GPU_BACKEND defaults to 'hip'
because gfx950 is the only target.  Assigning a value of another type raises
TypeError, an unknown key raises AttributeError, as in the reference.
"""
import os


class _Defaults:
    GPU_BACKEND = 'hip'
    HIPCC = 'hipcc'
    OFFLOAD_ARCH = 'gfx950'
    DEBUG = False
    SHOW_BUILDING_COMMAND = False
    # Where operator sources compiled on load keep their shared objects: beside the
    # source (`<operator>/build/`) or, with BUILD_IN_LOCAL_PATH False, under
    # `<BUILD_PATH>/build/<operator>_<hash of its parent directory>/`.
    BUILD_PATH = './'
    BUILD_IN_LOCAL_PATH = True
    # Device used to execute calls whose tensors live in host memory.
    HOST_STAGING_DEVICE = 0
    # Kept for source compatibility with scripts that set them; the HIP path
    # has no host thread team.
    USING_OPENMP = True
    HOST_NUM_THREADS = 0
    USING_ASYNC_EXEC = True
    # 'auto' | 'tiled' | 'naive': kernel family used by ROIAlign.
    ROIALIGN_IMPL = os.environ.get('MOBULA_ROIALIGN_IMPL', 'auto')


class Config:
    def __init__(self):
        for key in dir(_Defaults):
            if not key.startswith('_'):
                self.__dict__[key] = getattr(_Defaults, key)

    def __setattr__(self, key, value):
        if key not in self.__dict__:
            raise AttributeError("Config has no attribute '{}'".format(key))
        want, got = type(self.__dict__[key]), type(value)
        if want is not got:
            raise TypeError('The type of config attribute `{}` is not consistent, '
                            'target {} vs value {}.'.format(key, want, got))
        self.__dict__[key] = value


config = Config()


class TempConfig:
    """`with config.TempConfig(KEY=value): ...` restores the old values on exit."""

    def __init__(self, **overrides):
        self._new = overrides
        self._old = {}

    def __enter__(self):
        for key, value in self._new.items():
            if not hasattr(config, key):
                raise AttributeError("'mobula.config' object has no attribute '{}'".format(key))
            self._old[key] = getattr(config, key)
            setattr(config, key, value)
        return config

    def __exit__(self, *exc):
        for key, value in self._old.items():
            setattr(config, key, value)
        return False


Config.TempConfig = TempConfig

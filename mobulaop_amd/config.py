"""`mobula.config`: a bag of named settings, each with a fixed type.

Reading and writing are plain attribute access.  A setting that does not exist
raises AttributeError, a value whose type differs from the setting's raises
TypeError, and `mobula.config.TempConfig(NAME=value, ...)` is a context manager that
puts the old values back (reference: mobula/config.py:4-66; only the settings that
mean something on this build are kept, GPU_BACKEND is 'hip').
"""
import os

_SETTINGS = dict(
    GPU_BACKEND='hip',
    HIPCC='hipcc',
    OFFLOAD_ARCH='gfx950',
    DEBUG=False,
    SHOW_BUILDING_COMMAND=False,
    # Where operator sources compiled on load keep their shared objects: beside the
    # source (`<operator>/build/`) or, with BUILD_IN_LOCAL_PATH False, under
    # `<BUILD_PATH>/build/<operator>_<hash of its parent directory>/`.
    BUILD_PATH='./',
    BUILD_IN_LOCAL_PATH=True,
    # Device that executes calls whose tensors live in host memory.
    HOST_STAGING_DEVICE=0,
    # Accepted for scripts that set them; there is no host thread team here.
    USING_OPENMP=True,
    HOST_NUM_THREADS=0,
    USING_ASYNC_EXEC=True,
    # 'auto' | 'tiled' | 'naive': kernel family used by ROIAlign.
    ROIALIGN_IMPL=os.environ.get('MOBULA_ROIALIGN_IMPL', 'auto'),
)


class Config:
    def __init__(self, settings):
        self.__dict__.update(settings)

    def __setattr__(self, name, value):
        try:
            current = self.__dict__[name]
        except KeyError:
            raise AttributeError("Config has no attribute '{}'".format(name))
        if type(value) is not type(current):
            raise TypeError('The type of config attribute `{}` is not consistent, target {} vs value {}.'
                            .format(name, type(current), type(value)))
        self.__dict__[name] = value


config = Config(_SETTINGS)


class TempConfig:
    """`with TempConfig(NAME=value): ...`"""

    def __init__(self, **settings):
        self._wanted = settings
        self._saved = []

    def __enter__(self):
        for name, value in self._wanted.items():
            if name not in vars(config):
                raise AttributeError("'mobula.config' object has no attribute '{}'".format(name))
            self._saved.append((name, getattr(config, name)))
            setattr(config, name, value)
        return config

    def __exit__(self, *exc_info):
        while self._saved:
            setattr(config, *self._saved.pop())
        return False


Config.TempConfig = TempConfig

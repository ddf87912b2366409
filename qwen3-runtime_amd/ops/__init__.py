"""Device ops. ``HipOps`` is the only implementation the engine has."""


def __getattr__(name):
    if name in ("HipOps", "OpsError"):
        from . import hip

        return getattr(hip, name)
    raise AttributeError(name)

"""Backends created under particular environment settings (the library reads them when a backend is created)."""
import os


def backend_with_env(**env):
    from catgrad_amd import HipBackend

    old = {k: os.environ.get(k) for k in env}
    os.environ.update(env)
    try:
        return HipBackend(0)
    finally:
        for k, v in old.items():
            if v is None:
                del os.environ[k]
            else:
                os.environ[k] = v

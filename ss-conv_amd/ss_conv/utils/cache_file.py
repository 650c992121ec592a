"""On-disk cache of the pieces of the steerable basis (reference: ss_conv/utils/cache_file.py:49-112,
the decorator cached_dirpklgz used at utils/kernel.py:10 and utils/SO3.py:239).

The reference pickles results into ``cache/...`` under the current working directory, so the
files a process finds depend on where it was started.  Here the directory does not depend
on the working directory:

* ``set_cache_dir(path)`` chooses it for the process (``None`` switches the files off),
* else the environment variable ``SS_CONV_CACHE_DIR`` (empty, ``0`` or ``off``: no files),
* else ``$XDG_CACHE_HOME/ss_conv`` or ``~/.cache/ss_conv``.

Every result is one ``.npy`` file named after the function, its arguments and a format
version, written to a temporary name and moved into place (a reader never sees half a
file, and two writers of the same key leave one complete file), read back with
``numpy.load(allow_pickle=False)``: nothing in a cache file is executed.  A directory that
cannot be written, or a file that cannot be read, only costs the computation.
"""
import functools
import os
import tempfile

import numpy as np

FORMAT_VERSION = 1  # part of every file name: bump when a cached function changes its result

_UNSET = object()
_override = _UNSET
stats = {"computed": 0, "loaded": 0, "stored": 0}


def set_cache_dir(path):
    """Directory of the cache files for this process; None switches them off.  Results
    already held in memory stay."""
    global _override
    _override = None if path is None else os.path.abspath(os.fspath(path))


def cache_dir():
    """The directory in use, or None when files are switched off."""
    if _override is not _UNSET:
        return _override
    env = os.environ.get("SS_CONV_CACHE_DIR")
    if env is not None:
        return None if env.strip().lower() in ("", "0", "off", "none") else os.path.abspath(env)
    base = os.environ.get("XDG_CACHE_HOME") or os.path.join(os.path.expanduser("~"), ".cache")
    return os.path.join(base, "ss_conv")


def _file_of(name, args):
    d = cache_dir()
    if d is None:
        return None
    key = "_".join(str(a) for a in args)
    return os.path.join(d, name, "%s_v%d.npy" % (key, FORMAT_VERSION))


def cached_npy(name, maxsize=None):
    """Cache a function of hashable (integer) arguments that returns a numpy array: in
    memory for the life of the process and as ``<cache dir>/<name>/<args>_v<N>.npy``."""

    def decorator(func):
        @functools.lru_cache(maxsize=maxsize)
        @functools.wraps(func)
        def wrapper(*args):
            path = _file_of(name, args)
            if path is not None:
                try:
                    arr = np.load(path, allow_pickle=False)
                    stats["loaded"] += 1
                    return arr
                except (OSError, ValueError, EOFError):
                    pass
            arr = np.ascontiguousarray(func(*args))
            stats["computed"] += 1
            if path is not None:
                try:
                    os.makedirs(os.path.dirname(path), exist_ok=True)
                    fd, tmp = tempfile.mkstemp(dir=os.path.dirname(path), suffix=".tmp")
                    try:
                        with os.fdopen(fd, "wb") as f:
                            np.save(f, arr, allow_pickle=False)
                        os.replace(tmp, path)
                        stats["stored"] += 1
                    except BaseException:
                        try:
                            os.unlink(tmp)
                        except OSError:
                            pass
                        raise
                except OSError:
                    pass  # read-only or full file system: keep the result in memory only
            return arr

        return wrapper

    return decorator

"""Location of the on-disk caches (tuning records, code objects).

The reference keeps its downloaded performance models under the user cache
directory (spio/util/cache_dir.py, spio/kernels/performance_model_cache.py:46-56);
the tuning records of the on-device sweep live in the same kind of place.
SPIO_CACHE_DIR overrides it.
"""

import os


def get_cache_dir(*parts) -> str:
    """Return (and create) the cache directory, optionally a sub-directory."""
    root = os.environ.get("SPIO_CACHE_DIR")
    if not root:
        base = os.environ.get("XDG_CACHE_HOME") or os.path.join(os.path.expanduser("~"), ".cache")
        root = os.path.join(base, "spio_amd")
    path = os.path.join(root, *parts)
    os.makedirs(path, exist_ok=True)
    return path

"""Whether a built library matches its sources, judged by content and not by file times.

A build writes the SHA-256 of its source files and command line next to the library
(`<library>.srchash`).  A loader compares that stamp with the sources as they are now: file times do not
survive copying a tree to another machine, contents do.  A library without a stamp, or with another one,
is stale and its loader rebuilds it (a `RuntimeWarning` says so) unless PARPY_AMD_REBUILD=0 asks to load
what is there.
"""
import hashlib
import os
import warnings


def source_hash(paths, command):
    h = hashlib.sha256(" ".join(command).encode())
    for p in sorted(str(p) for p in paths):
        if os.path.exists(p):
            h.update(os.path.basename(p).encode())
            with open(p, "rb") as f:
                h.update(f.read())
    return h.hexdigest()


def stamp_path(lib):
    return str(lib) + ".srchash"


def write_stamp(lib, paths, command):
    with open(stamp_path(lib), "w") as f:
        f.write(source_hash(paths, command))


def is_current(lib, paths, command):
    try:
        with open(stamp_path(lib)) as f:
            return f.read().strip() == source_hash(paths, command)
    except OSError:
        return False


def ensure_current(lib, paths, command, build):
    """Make sure `lib` exists and matches `paths`; `build()` compiles it.  Returns True when it compiled."""
    if os.path.exists(str(lib)) and is_current(lib, paths, command):
        return False
    if os.path.exists(str(lib)):
        if os.environ.get("PARPY_AMD_REBUILD") == "0":
            warnings.warn(f"{os.path.basename(str(lib))} does not match its sources and PARPY_AMD_REBUILD=0 keeps it", RuntimeWarning)
            return False
        warnings.warn(f"{os.path.basename(str(lib))} does not match its sources: rebuilding it", RuntimeWarning)
    build()
    return True

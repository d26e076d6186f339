"""Persistent tile picker for the compiled HIP kernel instantiations.

Plays the role of reference src/trifast/autotune.py (``Autotuner.run``, :110-156)
and src/trifast/autotune_helpers.py, with the Triton config lists replaced by the
small set of tile instantiations compiled into ``libtrifast_hip.so``:

  * key      = ``H_DIM_CLOSESTN_dtype`` with ``CLOSEST_N = 2**ceil(log2 n)``
               (reference src/trifast/torch.py:45, autotune.py:114-120)
  * miss     = time every instantiation that supports the shape, keep the
               fastest, write the cache (reference autotune.py:121-137)
  * location = ``platformdirs.user_config_dir("trifast", version)``, one JSON file
               per kernel named ``{kernel}_{device-name}_{major}-{minor}.json``
               (reference autotune_helpers.py:22-37, autotune.py:73-75)
  * writes are tmp-file + ``os.replace`` under a lock; an unreadable cache is
    reported and ignored (reference autotune.py:83-108)
  * ``TRIFAST_FORCE_TUNE`` in {1,true,yes,on} re-tunes even on a hit
    (reference autotune_helpers.py:9-14, autotune.py:121)

``TRIFAST_AUTOTUNE=0`` turns timing off altogether: a miss then takes the
library's built-in heuristic pick and nothing is written.
"""

from __future__ import annotations

import json
import math
import os
import threading
from pathlib import Path
from typing import Callable

import torch

from trifast_amd import _lib

_TRUE = ("1", "true", "yes", "on")

FILE_LOCK = threading.Lock()


TIE_MARGIN = 1.02  # a tile must beat the default by more than this factor to replace it


def force_tune() -> bool:
    return os.getenv("TRIFAST_FORCE_TUNE", "0").lower() in _TRUE


def autotune_enabled() -> bool:
    return os.getenv("TRIFAST_AUTOTUNE", "1").lower() in _TRUE


def print_autotuning() -> bool:
    return os.getenv("TRIFAST_PRINT_AUTOTUNING", os.getenv("TRITON_PRINT_AUTOTUNING", "0")) == "1"


def get_config_dir() -> Path:
    import platformdirs

    from trifast_amd import __version__

    override = os.getenv("TRIFAST_CONFIG_DIR")
    path = Path(override) if override else Path(platformdirs.user_config_dir(appname="trifast", version=__version__))
    path.mkdir(parents=True, exist_ok=True)
    return path


def closest_n(n: int) -> int:
    return 2 ** int(math.ceil(math.log2(n))) if n > 1 else 1


def make_key(n: int, h: int, d: int, dtype: torch.dtype) -> str:
    return "_".join(map(str, (h, d, closest_n(n), dtype)))


def _device_tag(device=None) -> str:
    name = torch.cuda.get_device_name(device).replace(" ", "-").replace("/", "-")
    major, minor = torch.cuda.get_device_capability(device)
    return f"{name}_{major}-{minor}"


class TileCache:
    """key -> tile id of one kernel, mirrored in one JSON file."""

    def __init__(self, kernel: int):
        self.kernel = kernel
        self.name = _lib.KERNEL_NAMES[kernel]
        self.cache: dict[str, int] = {}
        self.cache_file: Path | None = None
        self.timings: dict[int, float] = {}
        try:
            self.cache_file = get_config_dir() / f"{self.name}_{_device_tag()}.json"
        except Exception as e:  # unwritable home etc.: tune in memory only
            print(f"Warning: no autotune cache directory: {e}")
        if self.cache_file is not None and self.cache_file.exists():
            try:
                with FILE_LOCK, open(self.cache_file, "rb") as f:
                    raw = json.load(f)
                for key, entry in raw.items():
                    tile = self._entry_to_tile(entry)
                    if tile is not None:
                        self.cache[key] = tile
            except Exception as e:
                print(f"Warning: Could not load autotune cache from {self.cache_file}: {e}")
                self.cache = {}

    def _tile_to_entry(self, tile: int) -> dict:
        info = _lib.tile_info(self.kernel, tile)
        return {
            "tile": tile,
            "kwargs": {"BLOCK_J": info["BLOCK_J"], "BLOCK_K": info["BLOCK_K"]},
            "num_waves": info["num_waves"],
        }

    def _entry_to_tile(self, entry) -> int | None:
        # an entry written for another build of the library (different tile table) is dropped
        try:
            tile = int(entry["tile"])
            if not 0 <= tile < _lib.load().trifast_num_tiles(self.kernel):
                return None
            return tile if self._tile_to_entry(tile) == entry else None
        except Exception:
            return None

    def write(self) -> None:
        if self.cache_file is None:
            return
        tmp = f"{self.cache_file}.{os.getpid()}.tmp"
        try:
            with FILE_LOCK:
                with open(tmp, "w") as f:
                    json.dump({k: self._tile_to_entry(t) for k, t in self.cache.items()}, f, indent=4)
                os.replace(tmp, self.cache_file)
        except Exception as e:
            print(f"Warning: Failed to write autotune cache: {e}")
        finally:
            if os.path.exists(tmp):
                os.remove(tmp)


_caches: dict[int, TileCache] = {}
_defaults: dict[tuple, int] = {}  # (kernel, n, h, d, dtype code) -> the library's heuristic pick


def _cache_for(kernel: int) -> TileCache:
    if kernel not in _caches:
        _caches[kernel] = TileCache(kernel)
    return _caches[kernel]


def reset() -> None:
    """Forget every in-memory cache (the files stay); used by tests."""
    _caches.clear()
    _defaults.clear()


def supported_tiles(kernel: int, n: int, h: int, d: int, dtype: torch.dtype) -> list[int]:
    lib = _lib.load()
    from trifast_amd.torch import _DTYPE_CODE

    code = _DTYPE_CODE[dtype]
    return [t for t in range(lib.trifast_num_tiles(kernel)) if lib.trifast_supports(kernel, t, n, h, d, code)]


def _time_launch(launch: Callable[[int], None], tile: int, warmup: int = 1, rep: int = 3) -> float:
    for _ in range(warmup):
        launch(tile)
    times = []
    for _ in range(rep):
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        launch(tile)
        end.record()
        end.synchronize()
        times.append(start.elapsed_time(end))
    times.sort()
    return times[len(times) // 2]


def pick(kernel: int, n: int, h: int, d: int, dtype: torch.dtype, launch: Callable[[int], None],
         extra_cost: Callable[[int], float] | None = None) -> int:
    """Tile id to run ``kernel`` with.  ``launch(tile)`` runs the kernel once on the
    caller's real arguments (outputs are overwritten by the caller's final launch).
    ``extra_cost(tile)`` is added to a tile's measured milliseconds: what the choice of
    that tile leaves for other kernels to do."""
    lib = _lib.load()
    from trifast_amd.torch import _DTYPE_CODE

    code = _DTYPE_CODE[dtype]

    def default() -> int:
        # (remembered per shape: at small sizes a step is bound by the host)
        dkey = (kernel, n, h, d, code)
        tile = _defaults.get(dkey)
        if tile is None:
            tile = lib.trifast_default_tile(kernel, n, h, d, code)
            _lib.check(min(tile, 0), "trifast_default_tile")
            _defaults[dkey] = tile
        return tile

    if not autotune_enabled() and not force_tune():
        return default()
    cache = _cache_for(kernel)
    key = make_key(n, h, d, dtype)
    if key in cache.cache and not force_tune():
        tile = cache.cache[key]
        if lib.trifast_supports(kernel, tile, n, h, d, code):
            return tile
    # timing synchronises with the device, which a stream capture (HIP graph,
    # torch.compile's reduce-overhead mode) does not survive: a miss under capture
    # takes the heuristic pick and leaves the cache alone
    if torch.cuda.is_available() and torch.cuda.is_current_stream_capturing():
        return default()
    tiles = supported_tiles(kernel, n, h, d, dtype)
    if not tiles:
        raise ValueError(f"no compiled tile of {cache.name} supports n={n} h={h} d={d} dtype={dtype}")
    if len(tiles) == 1:
        best = tiles[0]
        cache.timings = {}
    else:
        cache.timings = {t: _time_launch(launch, t) + (extra_cost(t) if extra_cost else 0.0) for t in tiles}
        best = min(cache.timings, key=cache.timings.get)
        # near-ties go to the library's default tile: timings of a few launches scatter by
        # a percent or two, and a stable choice is worth more than that
        default = lib.trifast_default_tile(kernel, n, h, d, code)
        if default in cache.timings and cache.timings[default] <= TIE_MARGIN * cache.timings[best]:
            best = default
    cache.cache[key] = best
    cache.write()
    if print_autotuning():
        print(f"trifast autotuning for {cache.name} key {key}: best tile {best} {_lib.tile_info(kernel, best)}; timings ms {cache.timings}")
    return best

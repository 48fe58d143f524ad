"""Compile and load ``libhipengine_gfx950.so``.

The library is built IN TREE (``hipengine_amd/lib``) by ``build_hip`` with
``hipcc --offload-arch=gfx950`` and opened with ``ctypes.CDLL``; a manifest next
to it records the content hash it was built from.  The planning half mirrors
hipEngine's ``hipengine/core/build.py`` (``plan_hip_build`` / ``build_hip``,
content-hash key over compiler, flags and source bytes, :911-932; env
``HIPENGINE_HIP_ARCH``, ``HIPENGINE_REQUIRE_CACHED_BUILD``, :17-24), without the
RDNA profiles (wave32, ``-mcumode``) that do not apply to gfx950.
"""

from __future__ import annotations

import ctypes
import hashlib
import os
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor
from dataclasses import dataclass, field
from pathlib import Path

_PACKAGE = Path(__file__).resolve().parents[1]
CSRC_DIR = _PACKAGE / "csrc"
LIB_DIR = _PACKAGE / "lib"
FAMILY = "hipengine_gfx950"
OUTPUT_NAME = "libhipengine_gfx950.so"
DEFAULT_ARCH = "gfx950"
_KEY_DOMAIN = "hipengine-gfx950-build-v1"

# -packed-fp32-ops is switched off on purpose: v_pk_{add,mul,fma}_f32 must not be
# generated for this target pool.
BASE_FLAGS: tuple[str, ...] = (
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
)


class BuildError(RuntimeError):
    pass


@dataclass(frozen=True)
class BuildArtifact:
    family: str
    key: str
    sources_digest: str
    sources: tuple[Path, ...]
    headers: tuple[Path, ...]
    flags: tuple[str, ...]
    compiler: str
    output: Path
    manifest: Path
    commands: tuple[tuple[str, ...], ...] = field(default=())

    @property
    def cached(self) -> bool:
        if not self.output.exists() or not self.manifest.exists():
            return False
        return self.manifest.read_text().split("\n", 1)[0].strip() == f"key={self.key}"


def target_arch() -> str:
    return os.environ.get("HIPENGINE_HIP_ARCH") or os.environ.get("HIPENGINE_HIP_OFFLOAD_ARCH") or DEFAULT_ARCH


def default_sources() -> tuple[Path, ...]:
    return tuple(sorted(CSRC_DIR.glob("*.hip")))


def default_headers() -> tuple[Path, ...]:
    return tuple(sorted(CSRC_DIR.glob("*.hpp"))) + tuple(sorted((_PACKAGE.parent / "include").glob("*.h")))


def _compiler() -> str:
    return os.environ.get("HIPENGINE_HIPCC") or shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


def _compiler_version(compiler: str) -> str:
    try:
        return subprocess.run([compiler, "--version"], check=True, capture_output=True, text=True).stdout
    except (OSError, subprocess.CalledProcessError):
        return "unknown"


def plan_hip_build(
    *,
    sources: tuple[Path, ...] | list[Path] | None = None,
    family: str = FAMILY,
    output_name: str = OUTPUT_NAME,
    extra_flags: tuple[str, ...] = (),
    compiler_version: str | None = None,
    out_dir: Path | None = None,
) -> BuildArtifact:
    """Describe the build without running it: key, flags, commands, output path."""
    srcs = tuple(Path(s) for s in (sources or default_sources()))
    hdrs = default_headers()
    compiler = _compiler()
    flags = BASE_FLAGS + (f"--offload-arch={target_arch()}",) + tuple(extra_flags)
    version = compiler_version if compiler_version is not None else _compiler_version(compiler)
    h = hashlib.sha256()
    for part in (_KEY_DOMAIN, Path(compiler).name, version, *flags):
        h.update(part.encode())
        h.update(b"\0")
    digest = sources_digest(srcs, hdrs)
    h.update(digest.encode())
    key = h.hexdigest()
    out = Path(out_dir) if out_dir else LIB_DIR
    obj_dir = out / "obj"
    commands = tuple(
        (compiler, *flags, "-c", str(s), "-o", str(obj_dir / (s.stem + ".o"))) for s in srcs
    ) + ((compiler, *flags, "-shared", *(str(obj_dir / (s.stem + ".o")) for s in srcs), "-o", str(out / output_name)),)
    return BuildArtifact(family, key, digest, srcs, hdrs, flags, compiler, out / output_name, out / "manifest.txt", commands)


def sources_digest(sources: tuple[Path, ...] | None = None, headers: tuple[Path, ...] | None = None) -> str:
    """sha256 over the names and bytes of the sources and headers the library is built from."""
    h = hashlib.sha256()
    for path in (*(sources or default_sources()), *(headers or default_headers())):
        h.update(path.name.encode())
        h.update(b"\0")
        h.update(path.read_bytes())
        h.update(b"\0")
    return h.hexdigest()


def write_manifest(art: BuildArtifact) -> None:
    art.manifest.write_text(
        f"key={art.key}\nsources_digest={art.sources_digest}\nfamily={art.family}\ncompiler={art.compiler}\n"
        f"flags={' '.join(art.flags)}\n" + "".join(f"source={s.name}\n" for s in art.sources)
    )


def _manifest_field(manifest: Path, name: str) -> str | None:
    if not manifest.exists():
        return None
    for line in manifest.read_text().splitlines():
        if line.startswith(name + "="):
            return line[len(name) + 1:].strip()
    return None


_loaded: dict[Path, ctypes.CDLL] = {}


def load_library(path: Path | None = None) -> ctypes.CDLL:
    """Open the built library (memoized).  Raises if it has not been built, or if the in-tree
    library was built from other sources than the ones next to it (a stale binary would silently
    be what runs): there is no other implementation to fall back to.  When a device is present the
    library's per-device set-up runs here, so that every entry point is graph-capturable from its
    first launch."""
    in_tree = path is None
    target = Path(path) if path else LIB_DIR / OUTPUT_NAME
    lib = _loaded.get(target)
    if lib is None:
        if not target.exists():
            raise BuildError(
                f"{target} is missing: build it with hipengine_amd.core.build.build_hip() "
                "(hipcc --offload-arch=gfx950); the gfx950 kernels have no CPU fallback"
            )
        if in_tree and os.environ.get("HIPENGINE_SKIP_STALE_CHECK") != "1":
            built_from = _manifest_field(target.parent / "manifest.txt", "sources_digest")
            if built_from != sources_digest():
                raise BuildError(
                    f"{target} is stale: its manifest records sources {str(built_from)[:16]}, the tree holds "
                    f"{sources_digest()[:16]}; rebuild with hipengine_amd.core.build.build_hip()"
                )
        lib = ctypes.CDLL(str(target))
        init = getattr(lib, "hipengine_gfx950_init", None)
        if init is not None:
            init.argtypes, init.restype = [], ctypes.c_int
            init()   # without a device this returns an error code and changes nothing; launches would fail anyway
        _loaded[target] = lib
    return lib


def build_hip(
    *,
    sources: tuple[Path, ...] | list[Path] | None = None,
    extra_flags: tuple[str, ...] = (),
    dry_run: bool = False,
    load: bool = True,
    require_cached: bool = False,
    force: bool = False,
    jobs: int = 4,
) -> ctypes.CDLL | BuildArtifact:
    """Compile (unless the manifest key matches) and optionally load the library."""
    art = plan_hip_build(sources=sources, extra_flags=extra_flags)
    if dry_run:
        return art
    need = force or not art.cached
    if need and (require_cached or os.environ.get("HIPENGINE_REQUIRE_CACHED_BUILD") == "1"):
        raise BuildError(f"{art.output} is not built for key {art.key[:16]} and compiling is disabled")
    if need:
        (art.output.parent / "obj").mkdir(parents=True, exist_ok=True)
        compile_cmds, link_cmd = art.commands[:-1], art.commands[-1]

        def run(cmd: tuple[str, ...]) -> None:
            proc = subprocess.run(cmd, capture_output=True, text=True)
            if proc.returncode != 0:
                raise BuildError(f"{' '.join(cmd)}\n{proc.stdout}\n{proc.stderr}")

        with ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
            list(pool.map(run, compile_cmds))
        run(link_cmd)
        write_manifest(art)
        _loaded.pop(art.output, None)
    return load_library(art.output) if load else art

"""Shared start-up of the command-line tools: compile the HIP library on first use (a fresh checkout holds sources only)."""
import os
import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent


def ensure_built() -> None:
    if (ROOT / "vllm-rust_amd" / "lib" / "libvmx.so").exists():
        return
    jobs = os.environ.get("MAX_JOBS") or str(min(16, os.cpu_count() or 4))
    print("building libvmx.so ...", file=sys.stderr, flush=True)
    subprocess.run(["make", "-C", str(ROOT / "vllm-rust_amd" / "csrc"), "-j" + jobs], check=True, stdout=sys.stderr)


def import_package():
    """Build if needed, then import the package from this checkout."""
    ensure_built()
    if str(ROOT) not in sys.path:
        sys.path.insert(0, str(ROOT))
    import vllm_rust_amd
    return vllm_rust_amd

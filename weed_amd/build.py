"""Build recipe for libweed_hip.so (hipcc, gfx950 only)."""
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
_CSRC = os.path.join(_HERE, "csrc")
_LIB = os.path.join(_HERE, "lib", "libweed_hip.so")
_HOST_LIB = os.path.join(_HERE, "lib", "libweed_host.so")


def library_path():
    """Path of libweed_hip.so; the environment variable WEED_HIP_LIBRARY overrides the in-tree build."""
    return os.environ.get("WEED_HIP_LIBRARY", _LIB)


def host_library_path():
    return _HOST_LIB


def build_library(force=True, jobs=8, verbose=False):
    """Compile every HIP source for gfx950 and link libweed_hip.so.  Raises on failure."""
    if force:
        subprocess.run(["make", "-C", _CSRC, "clean"], check=True, stdout=subprocess.DEVNULL)
    proc = subprocess.run(["make", "-C", _CSRC, "-j%d" % jobs, "all"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                          text=True)
    if verbose or proc.returncode:
        print(proc.stdout)
    if proc.returncode:
        raise RuntimeError("building libweed_hip.so failed (exit %d)" % proc.returncode)
    if not os.path.exists(_LIB):
        raise RuntimeError("make succeeded but %s is missing" % _LIB)
    return _LIB


def build_host(force=True, verbose=False):
    """Compile the host C++ mirror (weed_amd/host) into libweed_host.so; needs libweed_hip.so to link against."""
    host = os.path.join(_HERE, "host")
    if force:
        subprocess.run(["make", "-C", host, "clean"], check=True, stdout=subprocess.DEVNULL)
    proc = subprocess.run(["make", "-C", host, "all"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if verbose or proc.returncode:
        print(proc.stdout)
    if proc.returncode:
        raise RuntimeError("building libweed_host.so failed (exit %d)" % proc.returncode)
    return _HOST_LIB

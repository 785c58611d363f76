"""Native code of the tests, built with the package's own build module into tests/native/_lib (compiled
here if missing or stale; the build entry point compiles it beforehand):

* the toy plugin (tests/native/toy_plugin.hip): toy parts and architectures that are registered with the
  engine from outside the package. ``plugin_path()`` is the built library, ``load()`` hands it to the
  engine of this process;
* a kernel that exposes the lane exchanges of the kernels' common header (tests/native/lane_check.hip)."""
import os

from mini_llm_amd import build

HERE = os.path.dirname(os.path.abspath(__file__))

build.register_library("toy_plugin", {
    "kind": "plugin",
    "sources": [os.path.join(HERE, "native", "toy_plugin.hip")],
    "headers": [],
    "needs": ["engine"],                 # built after the engine library, which it links against
    "out_dir": os.path.join(HERE, "native", "_lib"),
})
build.register_library("lane_check", {
    "kind": "hip",
    "sources": [os.path.join(HERE, "native", "lane_check.hip")],
    "headers": [os.path.join(build.CSRC, "kernels", "common.h")],
    "out_dir": os.path.join(HERE, "native", "_lib"),
})
NATIVE = ("toy_plugin", "lane_check")


def plugin_path() -> str:
    if not build.is_current("toy_plugin"):
        build.build_library("toy_plugin")
    return build.lib_path("toy_plugin")


def load() -> str:
    import mini_llm_amd
    path = plugin_path()
    mini_llm_amd.load_plugin(path)
    return path

"""GPU: the replacement of the reference's AccCTR plugin (lib_ock_ctr_common.so, recsdk_amd/plugin) driven through
the reference's own interface: tests/plugin_driver.cpp loads it with ock::ctr::Factory::Create and runs cases modelled
on the reference's unit tests of Unique and EmbCacheManager.  Both are compiled against the reference's interface
headers (python -m recsdk_amd.plugin.build), which only a machine with a reference checkout can do; the built files
travel with the tree."""
import os
import subprocess

import pytest

from recsdk_amd.plugin import build as plugin_build

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("old_abi", [False, True])
def test_plugin_passes_the_reference_style_cases(old_abi):
    """old_abi: plugin and driver compiled with _GLIBCXX_USE_CXX11_ABI=0, as the reference builds AccCTR
    (AccCTR/src/CMakeLists.txt:30): the interface passes std::string and std::vector across the library boundary."""
    plugin = plugin_build.PLUGIN_OLD_ABI if old_abi else plugin_build.PLUGIN
    driver = plugin_build.DRIVER_OLD_ABI if old_abi else plugin_build.DRIVER
    out = plugin_build.OUT_OLD_ABI if old_abi else plugin_build.OUT
    if not (os.path.isfile(plugin) and os.path.isfile(driver)):
        if plugin_build.reference_includes() is None:
            pytest.skip("the plugin is not built and no reference checkout is here to build it against")
        plugin_build.build(old_abi=old_abi, verbose=False)
    env = dict(os.environ)
    env["LD_LIBRARY_PATH"] = out + os.pathsep + env.get("LD_LIBRARY_PATH", "")
    run = subprocess.run([driver], env=env, capture_output=True, text=True, timeout=300)
    tail = run.stdout[-4000:] + run.stderr[-2000:]
    assert run.returncode == 0, tail
    last = [ln for ln in run.stdout.splitlines() if ln.startswith("plugin_driver:")]
    assert last and last[-1].endswith(" 0 failures"), tail
    checks = int(last[-1].split()[1])
    assert checks > 200, tail

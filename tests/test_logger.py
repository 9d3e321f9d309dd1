"""The namespaced loggers and the memory report (the reference's yalis/logger.py:44-81,
yalis/utils.py:16-31)."""
import logging
import subprocess
import sys


def test_loggers_share_a_namespace_that_keeps_to_itself():
    from yalis_amd.utils.logger import get_logger, gpu_memory_info, max_gpu_memory_info

    a, b = get_logger("engine"), get_logger("weights")
    assert a.name == "yalis_amd.engine" and b.name == "yalis_amd.weights"
    root = logging.getLogger("yalis_amd")
    assert root.propagate is False and len(root.handlers) == 1, "configured once, whatever the number of loggers"
    alloc, reserved = gpu_memory_info()
    peak_alloc, peak_reserved = max_gpu_memory_info()
    assert 0 <= alloc <= reserved + 1e-9 and alloc <= peak_alloc + 1e-9 and reserved <= peak_reserved + 1e-9


def test_level_comes_from_the_environment():
    code = ("from yalis_amd.utils.logger import get_logger; l = get_logger('x'); "
            "l.info('quiet'); l.warning('loud'); l.debug('never')")
    for level, seen in (("WARNING", ["loud"]), ("INFO", ["quiet", "loud"]), ("", ["quiet", "loud"])):
        run = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, env={"YALIS_LOG_LEVEL": level, "PATH": "/usr/bin:/bin"},
                             cwd=__import__("os").path.dirname(__import__("os").path.dirname(__import__("os").path.abspath(__file__))))
        assert run.returncode == 0, run.stderr
        lines = [ln for ln in run.stderr.splitlines() if "yalis_amd.x:" in ln]
        assert [ln.rsplit(": ", 1)[1] for ln in lines] == seen
        assert all(ln.split()[1] in ("INFO", "WARNING") for ln in lines)

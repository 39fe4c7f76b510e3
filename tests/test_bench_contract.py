"""bench.py on a machine without a GPU: what can be checked of its command-line contract."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                         timeout=120)
    assert run.returncode != 0
    assert "one GPU" in run.stderr
    assert run.stdout.strip() == ""          # no JSON line for a run that did not happen


def test_help_lists_the_contract_flags():
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--help"], capture_output=True, text=True,
                         timeout=120)
    assert run.returncode == 0
    for flag in ("--gpus", "--steps", "--warmup"):
        assert flag in run.stdout


def _attributes_read(fn, name="args"):
    """Names of the attributes a function's source reads from its first parameter (`args.x`), nested functions included."""
    import ast
    import inspect
    import textwrap
    tree = ast.parse(textwrap.dedent(inspect.getsource(fn)))
    return {n.attr for n in ast.walk(tree)
            if isinstance(n, ast.Attribute) and isinstance(n.value, ast.Name) and n.value.id == name}


def test_the_legs_bench_starts_are_command_lines_config_bench_accepts():
    """bench.py runs the other configurations as `python -m recsdk_amd.config_bench --config cN --steps K --warmup W
    ...` in processes of their own: every planned command line must parse, and every option a configuration's function
    reads must be one the parser defines."""
    sys.path.insert(0, ROOT)
    import bench
    from recsdk_amd import config_bench as cb
    assert [p[0] for p in bench.OTHER_CONFIG_PLAN] == ["c1", "c3", "c4", "c5"]
    for name, steps, warmup, extra in bench.OTHER_CONFIG_PLAN:
        a = cb.make_parser().parse_args(["--config", name, "--steps", str(steps), "--warmup", str(warmup)] + list(extra))
        assert a.steps == steps and a.warmup == warmup and a.config == name
        fn_name = "run_" + name
        read = _attributes_read(getattr(cb, fn_name))
        assert read, fn_name
        missing = [x for x in read if not hasattr(a, x)]
        assert not missing, f"{fn_name} reads {missing}, which config_bench's parser does not define"
    # an override that names no option is refused instead of being carried silently
    import pytest
    with pytest.raises(AttributeError):
        cb.default_args(no_such_option=1)

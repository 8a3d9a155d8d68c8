"""Making `fp8_linear` known to hyper_parallel's operator dispatcher without losing its built-in operators.

The dispatcher reads exactly one directory of YAML files, once, when `hyper_parallel.core.shard._op_dispatch` is
imported (hyper_parallel/core/shard/_op_dispatch.py:96-99, :117-142, :613-632, singleton at :675):
HYPER_PARALLEL_OPS_YAML_DIR *replaces* the built-in `shard/ops/yaml` directory.  Pointing it at a directory that
holds only `fp8_linear_ops.yaml` would leave `linear`, `reshape`, `add` ... unregistered, and every one of them
would raise "dose not contain parallel layout infer func" (:657-658).  Two ways that keep them:

* before the import: `prepare_env()` builds a directory holding the built-in YAML files of the installed
  hyper_parallel package plus `fp8_linear_ops.yaml`, and sets the two environment variables;
* after the import: `register()` adds the one entry to the live dispatcher the way its own constructor would
  (`layout_infer_ops[name] = config`, then `_register_single_distributed_op`, :148-186).

Nothing here imports hyper_parallel unless `register()` is called without a dispatcher.
"""
from __future__ import annotations

import glob
import importlib
import importlib.util
import os
import shutil
import sys
import tempfile
from typing import Optional

import yaml

PLUGIN_DIR = os.path.dirname(os.path.abspath(__file__))
PLUGIN_YAML = os.path.join(PLUGIN_DIR, "fp8_linear_ops.yaml")
_DISPATCH_MODULE = "hyper_parallel.core.shard._op_dispatch"


def builtin_yaml_dir(hyper_parallel_dir: Optional[str] = None) -> str:
    """The directory of the installed hyper_parallel package that holds its built-in operator YAML files.  The
    package is located, not imported (importing it would construct the dispatcher and read the environment)."""
    if hyper_parallel_dir is None:
        spec = importlib.util.find_spec("hyper_parallel")
        if spec is None or not spec.submodule_search_locations:
            raise ModuleNotFoundError("hyper_parallel is not installed (or pass hyper_parallel_dir=)")
        hyper_parallel_dir = list(spec.submodule_search_locations)[0]
    d = os.path.join(hyper_parallel_dir, "core", "shard", "ops", "yaml")
    if not os.path.isdir(d):
        raise FileNotFoundError(f"no built-in operator YAML directory at {d}")
    return d


def merged_yaml_dir(dest: Optional[str] = None, hyper_parallel_dir: Optional[str] = None) -> str:
    """A directory holding copies of every built-in `*.yaml` plus `fp8_linear_ops.yaml`; returns its absolute path
    (a fresh temporary directory unless `dest` is given).  Raises if a built-in file already defines one of the
    plugin's operator names (the dispatcher itself refuses duplicates, _op_dispatch.py:627-629)."""
    src = builtin_yaml_dir(hyper_parallel_dir)
    dest = os.path.abspath(dest) if dest else tempfile.mkdtemp(prefix="hpfp8_ops_yaml_")
    os.makedirs(dest, exist_ok=True)
    ours = set(yaml.safe_load(open(PLUGIN_YAML, encoding="utf-8")))
    for f in sorted(glob.glob(os.path.join(src, "*.yaml"))):
        names = set(yaml.safe_load(open(f, encoding="utf-8")) or ())
        if names & ours:
            raise ValueError(f"{f} already defines {sorted(names & ours)}")
        shutil.copyfile(f, os.path.join(dest, os.path.basename(f)))
    shutil.copyfile(PLUGIN_YAML, os.path.join(dest, os.path.basename(PLUGIN_YAML)))
    return dest


def prepare_env(dest: Optional[str] = None, hyper_parallel_dir: Optional[str] = None, environ=None) -> str:
    """Set HYPER_PARALLEL_OPS_YAML_DIR (the merged directory) and HYPER_PARALLEL_OPS_PYTHON_PATH (this plugin's
    directory, appended to what is already there).  Must run before hyper_parallel's dispatcher module is imported;
    afterwards the variables are no longer read and this raises -- use `register()` then."""
    if _DISPATCH_MODULE in sys.modules:
        raise RuntimeError("hyper_parallel's dispatcher is already imported and has read its environment; "
                           "call hpfp8.plugin.install.register() instead")
    environ = os.environ if environ is None else environ
    d = merged_yaml_dir(dest, hyper_parallel_dir)
    environ["HYPER_PARALLEL_OPS_YAML_DIR"] = d
    paths = [p for p in environ.get("HYPER_PARALLEL_OPS_PYTHON_PATH", "").split(":") if p]
    if PLUGIN_DIR not in paths:
        paths.append(PLUGIN_DIR)
    environ["HYPER_PARALLEL_OPS_PYTHON_PATH"] = ":".join(paths)
    return d


def register(dispatcher=None) -> None:
    """Add `fp8_linear` to a dispatcher that already exists (default: hyper_parallel's singleton).  The plugin class
    is named by module (`distributed_op_module`), so no path variable is needed."""
    if dispatcher is None:
        dispatcher = importlib.import_module(_DISPATCH_MODULE)._OP_DISPATCHER
    for name, cfg in yaml.safe_load(open(PLUGIN_YAML, encoding="utf-8")).items():
        cfg = dict(cfg)
        cfg["distributed_op_module"] = __package__ + "." + cfg.pop("distributed_op_file")
        if name in dispatcher.layout_infer_ops:
            continue
        dispatcher.layout_infer_ops[name] = cfg
        dispatcher._register_single_distributed_op(name, cfg)


if __name__ == "__main__":
    d = merged_yaml_dir(sys.argv[1] if len(sys.argv) > 1 else None)
    print(f"export HYPER_PARALLEL_OPS_YAML_DIR={d}")
    print(f"export HYPER_PARALLEL_OPS_PYTHON_PATH={PLUGIN_DIR}")

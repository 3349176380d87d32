"""MI355X-native Evoformer hot path behind the interface of ``fastfold.model.fastnn``."""


def install_as_fastfold():
    """Opt-in alias: after this call ``import fastfold.model.fastnn``, ``from fastfold.distributed import ...`` and
    ``from fastfold.utils.inject_fastnn import inject_fastnn`` resolve to this package's modules, so scripts written
    against the reference (e.g. ``from fastfold.model.fastnn import Evoformer``, benchmark/perf.py:7-8) run
    unedited.  Refuses to shadow a real ``fastfold`` package that is already imported."""
    import importlib
    import pkgutil
    import sys

    me = sys.modules[__name__]
    have = sys.modules.get("fastfold")
    if have is not None and have is not me:
        raise RuntimeError("install_as_fastfold: another 'fastfold' package is already imported (%r)"
                           % getattr(have, "__file__", have))
    names = [__name__]
    for info in pkgutil.walk_packages(me.__path__, prefix=__name__ + "."):
        if ".csrc" in info.name:            # the kernel sources and their build script are not part of the surface
            continue
        names.append(info.name)
    for name in names:
        sys.modules["fastfold" + name[len(__name__):]] = importlib.import_module(name)
    return me

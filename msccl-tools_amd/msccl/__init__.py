"""msccl for MI355X: MSCCLang (msccl.language), the plan registry (msccl.init) and the executor that
runs compiled MSCCL-IR on one MI355X through the HIP library libmscclx.so (msccl.executor)."""
__version__ = "0.1.0"


def __getattr__(name):
    # msccl.init / msccl.Collective / plan listing, loaded on first use
    if name in ("init", "Collective", "tabulate_plans", "print_plans"):
        from msccl import autosynth
        return getattr(autosynth, name)
    raise AttributeError(name)

"""An inference engine for one AMD Instinct MI355X: typed configurations, safetensors weights,
layers built from parts, a paged cache, one step function, a scheduler and sampling, on
hand-written HIP kernels for gfx950.  Imported as `geneinfer_amd`."""
__version__ = "0.1.0"


def __getattr__(name):
    # The public names are loaded on first use so that `import geneinfer_amd.config` stays light.
    import importlib
    api = importlib.import_module("geneinfer_amd.api")
    public = {"LLM": api.LLM, "Engine": api.Engine, "EngineConfig": api.EngineConfig, "EngineRequest": api.EngineRequest,
              "Runner": api.Runner, "SamplerConfig": api.SamplerConfig, "Sampler": api.Sampler, "generate": api.generate,
              "load_model": api.load_model, "random_model": api.random_model}
    if name in public:
        return public[name]
    raise AttributeError(f"module 'geneinfer_amd' has no attribute {name!r}")

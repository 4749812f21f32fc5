"""An inference engine for one AMD Instinct MI355X: typed configurations, safetensors weights,
layers built from parts, a paged cache, one step function, a scheduler and sampling, on
hand-written HIP kernels for gfx950.  Imported as `geneinfer_amd`."""
__version__ = "0.1.0"

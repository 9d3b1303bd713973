"""HIP kernels of the engine: `build` compiles them, `library` calls them."""

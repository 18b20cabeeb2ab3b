from .module_cache import ModuleCache, build_kernel_function_name, compile_functions  # noqa: F401

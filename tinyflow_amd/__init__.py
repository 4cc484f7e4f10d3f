"""tinyflow_amd: MI355X-native training hot path behind tinyflow's DLArray C-ABI.

Modules mirror the reference package ``pycode/tinyflow`` for the hot path only:
``ndarray`` (array container), ``gpu_op`` (one wrapper per C entry point),
``autodiff`` (graph, reverse-mode gradients) and ``TrainExecute`` (SGD step
executor).  Importing the package loads ``lib/libc_runtime_api.so``; there is no
CPU fallback - without the library the import raises.
"""

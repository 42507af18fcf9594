"""heron_amd - MI355X (gfx950) backend for the tensor programs the Heron auto-scheduler tunes.

Layout mirrors the reference package so that a Heron user finds the same names:
``ops/rocm`` (operator definitions), ``task``, ``schedule/{context,sched_op,constraints}``,
``tuner``, ``model``, ``runner``, ``perf``, ``environment``, ``config``, ``sample``, ``multi``.
The kernels themselves are HIP templates under ``csrc/`` behind the C ABI of
``include/heron_rocm.h``; ``backend`` is the ctypes binding.
"""
__version__ = "0.1.0"

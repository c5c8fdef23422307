"""Registration of the custom-call targets with JAX-on-ROCm.

Counterpart of brainpylib/_src/register_custom_calls.py:10-22: every capsule of
``gpu_ops.registrations()`` is handed to XLA under its target name.  On a ROCm build of jaxlib the
platform string is "ROCM" (the reference registers under "gpu", which current jaxlib maps to CUDA).

Nothing in this package imports this module; call ``register()`` from an environment that has
jax installed.  It raises ImportError otherwise.
"""


def register(platform="ROCM"):
  """Registers all targets; returns their names."""
  from jax.lib import xla_client  # noqa: F401  (ImportError if jax is absent)
  from . import gpu_ops
  names = []
  for name, capsule in gpu_ops.registrations().items():
    try:
      xla_client.register_custom_call_target(name, capsule, platform=platform)
    except TypeError:  # jaxlib spellings differ between releases
      xla_client.register_custom_call_target(name.encode(), capsule, platform)
    names.append(name)
  return names

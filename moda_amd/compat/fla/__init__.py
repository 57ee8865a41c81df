"""Import-path shim: put ``moda_amd/compat`` on ``sys.path`` and model code that does
``from fla.ops.moda import parallel_moda`` (vision_tasks/deit/models.py:12) resolves to the HIP operators."""

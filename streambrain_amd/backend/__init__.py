"""Backend modules of the package; `hip_backend` is the one BCPNN_BACKEND=hip selects."""

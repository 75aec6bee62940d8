"""Python modules with the names and call signatures of the reference's pybind
extensions (`fchl_gpu`, `pairlist_gpu`, `sorf_gpu`, `rff_gpu`, `utils_gpu`;
reference setup.py:37-117), implemented over libqmll."""

"""MI355X-native drop-in for the Muon orthogonalisation path of Emerging-Optimizers.

Module paths, function names and signatures follow the reference package so that existing imports
(``from emerging_optimizers.orthogonalized_optimizers import muon_utils`` ...) keep working once this
directory is first on ``sys.path``.  The device work is done by hand-written gfx950 kernels in
``csrc/`` reached through ``_hip`` (ctypes over a C ABI); see ``hip_kernels``.
"""

__version__ = "0.1.0"

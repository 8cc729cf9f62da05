"""MI355X-native Muon / MuonH optimizer hot path (hand-written gfx950 HIP kernels behind a C ABI).

``archscale_amd.optim``     mirrors ``lit_gpt.optim`` of the reference (Muon / MuonH, Newton-Schulz hooks)
``archscale_amd.emerging``  mirrors ``emerging_optimizers.orthogonalized_optimizers`` (OrthogonalizedOptimizer, Muon)
"""
__version__ = "0.1.0"

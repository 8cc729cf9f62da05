"""Mirror of the reference's ``lit_gpt/optim`` for MI355X.

Submodules: ``muon`` (the optimizer), ``newton_schulz_hip`` (Newton-Schulz hooks and single products),
``opt_utils`` (parameter batching).  Import the hooks from their submodule, as with the reference.
"""

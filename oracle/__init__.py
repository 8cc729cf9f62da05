"""CPU oracle for the Muon / MuonH optimizer hot path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``archscale_amd/`` may import this
package: it exists so that tests, the smoke check and the benchmark's CPU
baseline leg have an independent statement of what the HIP path must compute.
"""

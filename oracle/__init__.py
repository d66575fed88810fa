"""CPU restatement of the reference's streaming-attention semantics.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this
module: it exists so that tests, the smoke check and the benchmark's CPU
baseline have an independent statement of what the operator must compute.
"""

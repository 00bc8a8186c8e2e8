"""CPU oracle for the pipeline-stage hot path. TEST INFRASTRUCTURE ONLY.

Nothing shipped imports this package: it is the checker that tests, the smoke
check and the bench's CPU-baseline leg compare the HIP stage against.
"""

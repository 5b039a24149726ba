"""CPU restatement of the reference operator layer.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory: it exists so that parity tests, the smoke check and the
``cpu_baseline`` leg of the benchmark have an independent, slow, readable
statement of what every operator must compute.
"""

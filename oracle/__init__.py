"""CPU oracle for the ChunkAttention decode path: TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this
package, and only as the checker -- never as the thing measured as the product or shipped.
"""

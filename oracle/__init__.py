"""CPU oracle for the MoE-layer + flat-buffer AdamW hot path.

TEST INFRASTRUCTURE ONLY.  Nothing under the product package may import this
package; only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg do,
and there only as the checker / the reported CPU baseline.
"""

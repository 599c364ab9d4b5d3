"""TEST INFRASTRUCTURE ONLY.  CPU restatements of the operations on the
generated-kernel path, used as the checker by tests/, __graft_entry__.smoke()
and the cpu_baseline leg of bench.py.  Nothing under cupy_amd/ imports this
package."""

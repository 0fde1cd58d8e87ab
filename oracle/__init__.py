"""CPU oracle for the gradient codec - TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may import this
package.  The product (templar_amd) never does and fails loudly without its HIP library.

`codec` wraps liborc.so (tplr_oracle.c, plain C, one function per reference routine);
`torch_cpu_path` issues the reference's own sequence of torch CPU ops and is what the
benchmark times as the CPU baseline.
"""

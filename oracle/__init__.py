"""CPU oracle for the quantized-contraction path. Test infrastructure only: the shipped
package (hipkittens_amd) never imports this; tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py do."""

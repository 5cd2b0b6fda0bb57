"""CPU oracle for the SparseDrop hot path.  Test infrastructure: imported only by tests/, the smoke
check and the cpu_baseline leg of bench.py — never by the flash_dropout package."""

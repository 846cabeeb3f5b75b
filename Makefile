# Convenience targets; everything they do is also reachable as the python commands shown.
PYTHON ?= python

.PHONY: build oracle test test-gpu bench sweep clean

build:            ## hipcc --offload-arch=gfx950 -> tccl_amd/libtccl_amd.so, plus the C client
	$(PYTHON) -m tccl_amd.build

oracle:           ## the CPU oracle used by the tests
	$(MAKE) -C oracle

test: build oracle  ## everything that needs no GPU
	$(PYTHON) -m pytest tests -x -q -m "not gpu"

test-gpu:         ## bit-exact parity on an MI355X (library must be built)
	$(PYTHON) -m pytest tests -x -q -m gpu

bench:            ## one JSON line: W=8 x 64 MiB bf16 all-reduce, the other ops and the size sweep
	$(PYTHON) bench.py

sweep:            ## one operation alone, e.g. make sweep OP=reduce_scatter_bf16
	$(PYTHON) bench.py --only $(OP)

clean:
	rm -rf tccl_amd/csrc/_obj tccl_amd/libtccl_amd.so tests/c_client/build
	$(MAKE) -C oracle clean

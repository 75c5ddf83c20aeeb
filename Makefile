# Task runner with the reference's target names (reference Makefile:12-61), for gfx950.
SHELL := /bin/bash
KERNELS ?= all
PYTHON ?= python

setup:
	mkdir -p logs profiles
	KERNELS=cublas_gemm $(PYTHON) compile_kernels.py build_ext --inplace

compile:
	KERNELS=$(KERNELS) $(PYTHON) compile_kernels.py build_ext --inplace

run:
	mkdir -p logs
	$(PYTHON) bench.py > ./logs/bench.log 2>&1

try:;$(MAKE) compile;$(MAKE) run

# the reference's harness flow (its bench.py) with its environment controls KERNELS / TEST_GEMM / PROFILING
harness:
	KERNELS=$(if $(filter all,$(KERNELS)),s2_128,$(KERNELS)) $(PYTHON) -m vq_gemm_amd.harness

# every kernel variant timed on one shape, next to the automatic choice: make tune SHAPE="512 4096 4096"
SHAPE ?= 512 4096 4096 8 256 32 8
tune:
	$(PYTHON) -m vq_gemm_amd.tune $(SHAPE)

test:
	$(PYTHON) -m pytest tests -x -q -m "not gpu"

test-gpu:
	$(PYTHON) -u -m pytest tests -x -v -m gpu --timeout 120 --timeout-method thread

# rocprofv3 takes the place of the reference's ncu target (reference Makefile:26-28)
profile:
	mkdir -p build/prof
	cd /tmp && TMPDIR=/tmp rocprofv3 --kernel-trace --stats --output-format csv -d $(CURDIR)/build/prof -o bench -- python3 $(CURDIR)/bench.py

clean:
	@rm -rf build vq_gemm_amd/lib oracle/libvq_oracle.so

.PHONY: setup compile run try harness tune test test-gpu profile clean

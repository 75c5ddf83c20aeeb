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

# one launch of one module under the profiler: the reference's per-variant targets (reference Makefile:24-28,53-57)
prof-harness:
	mkdir -p build/prof
	cd /tmp && TMPDIR=/tmp PROFILING=TRUE KERNELS=$(KERNELS) PYTHONPATH=$(CURDIR) rocprofv3 --kernel-trace --stats --output-format csv -d $(CURDIR)/build/prof -o $(KERNELS) -- python3 -m vq_gemm_amd.harness

# per-variant shorthands with the reference's names (reference Makefile:36-61)
VARIANTS := s1 s2_128 s2_512 s3_naive s3_wasp
define variant_targets
try-$(subst _,-,$(1)):;$$(MAKE) compile KERNELS=$(1) && $$(MAKE) harness KERNELS=$(1)
run-$(subst _,-,$(1)):;$$(MAKE) harness KERNELS=$(1)
prof-$(subst _,-,$(1)):;$$(MAKE) prof-harness KERNELS=$(1)
endef
$(foreach v,$(VARIANTS),$(eval $(call variant_targets,$(v))))
run-gemm-128:;TEST_GEMM=TRUE $(MAKE) harness KERNELS=s1
run-gemm-s2:;TEST_GEMM=TRUE $(MAKE) harness KERNELS=s2_128

clean:
	@rm -rf build vq_gemm_amd/lib oracle/libvq_oracle.so figures

.PHONY: setup compile run try harness tune test test-gpu profile prof-harness clean run-gemm-128 run-gemm-s2

# MI355X (gfx950) backend of the iris attention hot path.
#
#   make rocm     -> iris_c_amd/libiris_dev.so   (host C + HIP kernels, C ABI of include/iris_dev.h)
#   make oracle   -> oracle/*.so                  (CPU checker; test infrastructure)
#   make test-cpu / test-gpu / bench
ROCM_HOME ?= /opt/rocm
HIPCC     ?= $(ROCM_HOME)/bin/hipcc
CC        ?= gcc
CXX       ?= g++
GPU_ARCH  ?= gfx950

CSRC   = iris_c_amd/csrc
OUT    = iris_c_amd/libiris_dev.so
# Packed-f32 instruction selection is switched off for all device code.
HIPFLAGS = -O3 --offload-arch=$(GPU_ARCH) -fPIC -std=c++17 -Xclang -target-feature -Xclang -packed-fp32-ops \
           -I$(CSRC) -Iinclude
# gcc/g++ read the HIP runtime's host headers: they want the platform named on the command line
HOSTDEFS = -D__HIP_PLATFORM_AMD__=1
CFLAGS   = -O2 -fPIC -Wall -Wextra -std=c11 $(HOSTDEFS) -I$(CSRC) -Iinclude -I$(ROCM_HOME)/include

HIP_SRCS = $(CSRC)/qknorm_rope.hip $(CSRC)/fa_fwd_gfx950.hip $(CSRC)/fa_fwd_hd512_gfx950.hip $(CSRC)/attn_generic.hip \
           $(CSRC)/ew_norm_ops.hip $(CSRC)/gemm_conv_gfx950.hip $(CSRC)/rope_tables.hip
HIP_OBJS = $(HIP_SRCS:.hip=.o)
HOST_HDRS = include/iris_dev.h include/iris_rope.h $(CSRC)/iris_kernels_hip.h $(CSRC)/iris_rope_internal.h

.PHONY: rocm oracle clean test-cpu test-gpu bench ctest path pathcheck
rocm: $(OUT) iris_c_amd/libiris_microbench.so

# The hot path alone, for a host backend that keeps everything else (its own init, memory entries, stream and the
# other operators): the attention and norm+rope kernels and their two dispatch functions, none of the setup /
# memory / operator symbols that would clash with the host's.
PATH_LIB = iris_c_amd/libiris_dev_path.a
path: $(PATH_LIB)
$(CSRC)/iris_rocm_path.o: $(CSRC)/iris_rocm.c $(HOST_HDRS)
	$(CC) $(CFLAGS) -DIRIS_DEV_PATH_ONLY -c $< -o $@
$(PATH_LIB): $(CSRC)/qknorm_rope.o $(CSRC)/fa_fwd_gfx950.o $(CSRC)/fa_fwd_hd512_gfx950.o $(CSRC)/attn_generic.o $(CSRC)/iris_rocm_path.o
	rm -f $@ && ar rcs $@ $^
# link check: a host program that defines its OWN iris_dev_init / alloc / ... (as the reference's backend object
# does) next to the archive: no duplicate symbols, the hot-path calls resolve to the archive
pathcheck: tests/path_only_link.bin
tests/path_only_link.bin: tests/path_only_link.c include/iris_dev.h include/iris_dev_path.h $(PATH_LIB)
	$(CC) -O2 -Wall -Wextra -std=c11 $(HOSTDEFS) -Iinclude -I$(ROCM_HOME)/include -c $< -o tests/path_only_link.o
	$(HIPCC) --offload-arch=$(GPU_ARCH) -o $@ tests/path_only_link.o $(PATH_LIB) -L$(ROCM_HOME)/lib -lamdhip64 -lm \
	    -Wl,-rpath,$(ROCM_HOME)/lib

# C-language parity program: host C over the ABI, checked against the oracle (run by the GPU tests)
ctest: tests/c_abi_parity.bin
tests/c_abi_parity.bin: tests/c_abi_parity.c include/iris_dev.h include/iris_rope.h oracle/iris_oracle.h $(OUT) oracle/libiris_oracle.so
	$(CC) -O2 -Wall -Wextra -std=c11 -Iinclude -Ioracle -o $@ $< -Liris_c_amd -liris_dev -Loracle -liris_oracle \
	    -Wl,-rpath,'$$ORIGIN/../iris_c_amd' -Wl,-rpath,'$$ORIGIN/../oracle' -Wl,-rpath,$(ROCM_HOME)/lib -lm

oracle/libiris_oracle.so:
	$(MAKE) -C oracle oracle

# machine-ceiling microbenchmarks used by bench.py only
iris_c_amd/libiris_microbench.so: $(CSRC)/microbench.hip
	$(HIPCC) $(HIPFLAGS) -shared -o $@ $<

$(CSRC)/%.o: $(CSRC)/%.hip $(CSRC)/iris_kernels_hip.h $(CSRC)/norm_rope_math.h
	$(HIPCC) $(HIPFLAGS) -c $< -o $@

$(CSRC)/iris_rocm.o: $(CSRC)/iris_rocm.c $(HOST_HDRS)
	$(CC) $(CFLAGS) -c $< -o $@

# host builders of the rotary tables: IEEE arithmetic (no -ffast-math), their values are compared bit for bit
$(CSRC)/iris_rope_tables.o: $(CSRC)/iris_rope_tables.c $(HOST_HDRS)
	$(CC) $(CFLAGS) -c $< -o $@

# glue to the vendor GEMM library: host C++ only; the library itself is opened with dlopen at run time
$(CSRC)/linear_hipblaslt.o: $(CSRC)/linear_hipblaslt.cpp $(CSRC)/iris_kernels_hip.h
	$(CXX) -O2 -fPIC -Wall -Wextra -std=c++17 $(HOSTDEFS) -I$(CSRC) -I$(ROCM_HOME)/include -c $< -o $@

$(OUT): $(HIP_OBJS) $(CSRC)/iris_rocm.o $(CSRC)/iris_rope_tables.o $(CSRC)/linear_hipblaslt.o
	$(HIPCC) --offload-arch=$(GPU_ARCH) -shared -o $@ $^ -L$(ROCM_HOME)/lib -lamdhip64 -lm -ldl

oracle:
	$(MAKE) -C oracle all

test-cpu:
	python -m pytest tests -x -q -m "not gpu"
test-gpu:
	python -u -m pytest tests -x -v -m gpu --timeout 120 --timeout-method thread
bench:
	python bench.py

clean:
	rm -f $(CSRC)/*.o $(OUT) $(PATH_LIB) iris_c_amd/libiris_microbench.so tests/c_abi_parity.bin tests/path_only_link.bin tests/path_only_link.o

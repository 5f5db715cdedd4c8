# MI355X-native openfish: static library for callers of the openfish C API
# (lib/libopenfish.a, the artefact the reference Makefile produces with rocm=1)
# and a shared library with the same symbols for ctypes-based tests and benches
# (openfish_amd/libopenfish_amd.so).
#
#   make            both libraries
#   make rocm=1     accepted for compatibility with the reference's invocation
#   make oracle     the CPU oracle used by the tests (never linked into the libraries)
#   ./openfish <scores.blob> <N> <state_len>   decode a blob, write moves/sequence/qstring.blob

ROCM_ROOT ?= /opt/rocm
HIPCC     ?= $(ROCM_ROOT)/bin/hipcc
CC        ?= gcc
AR        ?= ar
ROCM_ARCH ?= --offload-arch=gfx950

SRC   := openfish_amd/csrc
BUILD := build
# -ffp-contract=off: every fp32 product and sum rounds separately, as on the CPU path.
# packed fp32 instructions are disabled for the whole device build.
HIPFLAGS := $(ROCM_ARCH) -O3 -fPIC -ffp-contract=off -Xclang -target-feature -Xclang -packed-fp32-ops \
            -Wall -Wno-unused-command-line-argument -I include -I $(SRC)
CFLAGS   := -O2 -g -Wall -fPIC -std=gnu11 -D__HIP_PLATFORM_AMD__ -I include -I $(SRC) -I $(ROCM_ROOT)/include
LDLIBS   := -L$(ROCM_ROOT)/lib -Wl,-rpath,$(ROCM_ROOT)/lib -lamdhip64 -lm -lpthread

HIP_OBJ := $(BUILD)/scan.o $(BUILD)/scan_five.o $(BUILD)/beam.o $(BUILD)/sequence.o $(BUILD)/rotary.o $(BUILD)/copy.o $(BUILD)/probe.o
C_OBJ   := $(BUILD)/openfish_host.o

all: lib/libopenfish.a openfish_amd/libopenfish_amd.so openfish

$(BUILD)/%.o: $(SRC)/%.hip $(SRC)/kernels.h $(SRC)/dmath.h
	@mkdir -p $(BUILD)
	$(HIPCC) $(HIPFLAGS) -c $< -o $@

# the scans once more for scores with five columns per state (a blank first), read in place
$(BUILD)/scan_five.o: $(SRC)/scan.hip $(SRC)/kernels.h $(SRC)/dmath.h
	@mkdir -p $(BUILD)
	$(HIPCC) $(HIPFLAGS) -DOFK_COLS=5 -c $< -o $@

$(BUILD)/%.o: $(SRC)/%.c $(SRC)/kernels.h include/openfish/openfish.h include/openfish/openfish_amd.h include/openfish/openfish_error.h
	@mkdir -p $(BUILD)
	$(CC) $(CFLAGS) -c $< -o $@

lib/libopenfish.a: $(HIP_OBJ) $(C_OBJ)
	@mkdir -p lib
	rm -f $@
	$(AR) rcs $@ $^

openfish_amd/libopenfish_amd.so: $(HIP_OBJ) $(C_OBJ)
	$(HIPCC) $(ROCM_ARCH) -shared -fPIC $^ -o $@ $(LDLIBS)

# the command-line driver (the reference's `openfish` test binary), linked against the static library
openfish: $(SRC)/openfish_cli.c lib/libopenfish.a
	$(CC) $(CFLAGS) $< lib/libopenfish.a $(LDLIBS) -lstdc++ -o $@

oracle:
	$(MAKE) -C oracle

clean:
	rm -rf $(BUILD) lib/libopenfish.a openfish_amd/libopenfish_amd.so openfish

.PHONY: all oracle clean

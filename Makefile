# Build and check the MI355X (gfx950) library without Python in the loop.
#   make            libmegagemm_hip.so, the CPU oracle and the standalone check
#   make run        run the standalone check on the GPU (exit code = outcome)
#   make test       CPU test-suite
#   make clean
HIPCC   ?= /opt/rocm/bin/hipcc
PYTHON  ?= python3
LIB      = mgrrmsnorm_amd/libmegagemm_hip.so
ORACLE   = oracle/libmg_oracle.so
CHECK    = tests/standalone/rmsnorm_standalone

all: $(LIB) $(ORACLE) $(CHECK)

$(LIB): $(wildcard mgrrmsnorm_amd/csrc/*.hip mgrrmsnorm_amd/csrc/*.hpp include/*.h)
	$(PYTHON) -m mgrrmsnorm_amd._build

$(ORACLE): oracle/mg_oracle.c
	$(MAKE) -C oracle libmg_oracle.so

$(CHECK): tests/standalone/rmsnorm_standalone.cpp include/megagemm_hip.h $(LIB) $(ORACLE)
	$(HIPCC) -O2 -std=c++17 -Iinclude $< -o $@ \
	    -Lmgrrmsnorm_amd -lmegagemm_hip -Loracle -lmg_oracle \
	    -Wl,-rpath,'$$ORIGIN/../../mgrrmsnorm_amd' -Wl,-rpath,'$$ORIGIN/../../oracle'

run: $(CHECK)
	./$(CHECK)

test:
	$(PYTHON) -m pytest tests -q -m "not gpu"

clean:
	rm -rf $(LIB) $(ORACLE) $(CHECK) mgrrmsnorm_amd/csrc/_obj

.PHONY: all run test clean

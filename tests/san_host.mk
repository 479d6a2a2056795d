# Builds tests/san_host and tests/_san/libsan_host.so: the host side of the library under sanitizers, on the CPU
# (tests/test_host_sanitizers.py runs `make -f san_host.mk san_host`).  Kept apart from tests/Makefile because
# nothing here is for a machine with a GPU.
# The two host translation units of the library under ASan and UBSan (host code only: the device side of
# eri_optim8_api.cpp is compiled as it always is), in front of the product library, and the program that drives
# them.  Both with the clang of the ROCm tree, whose sanitizer runtime they share.
CLANGXX := /opt/rocm/lib/llvm/bin/clang++
HIPCC   ?= /opt/rocm/bin/hipcc
SAN     := -fsanitize=address -fsanitize=undefined -fno-omit-frame-pointer
CSRC    := ../eridiffusion_amd/csrc
SANRT   := $(dir $(shell $(CLANGXX) -print-file-name=libclang_rt.asan-x86_64.so))

_san/libsan_host.so: $(CSRC)/eri_optim8_api.cpp $(CSRC)/eri_adam8bit_host.cpp $(CSRC)/eri_adam8_device.h ../include/eri_optim8.h ../include/eri_adam8bit.h ../eridiffusion_amd/liberi_optim8.so
	mkdir -p _san
	$(HIPCC) -O1 -g -fPIC -std=c++17 -ffp-contract=off --offload-arch=gfx950 -Xclang -target-feature -Xclang -packed-fp32-ops \
	    -Xarch_host -fsanitize=address -Xarch_host -fsanitize=undefined -Xarch_host -fno-omit-frame-pointer -x hip -c $(CSRC)/eri_optim8_api.cpp -o _san/api.o
	$(CLANGXX) -O1 -g -fPIC -std=c++17 $(SAN) -c $(CSRC)/eri_adam8bit_host.cpp -o _san/host.o
	$(HIPCC) -shared -fPIC --offload-arch=gfx950 _san/api.o _san/host.o -o $@ -fsanitize=address -fsanitize=undefined -shared-libsan \
	    -L../eridiffusion_amd -leri_optim8 -Wl,-rpath,'$$ORIGIN/../../eridiffusion_amd' -Wl,-rpath,/opt/rocm/lib -Wl,-rpath,$(SANRT)

san_host: san_host.cpp _san/libsan_host.so ../include/eri_optim8.h ../include/eri_adam8bit.h
	$(CLANGXX) -O1 -g -std=c++17 $(SAN) -shared-libsan -I../include $< -o $@ -L_san -lsan_host -L../eridiffusion_amd -leri_optim8 \
	    -Wl,-rpath,'$$ORIGIN/_san' -Wl,-rpath,'$$ORIGIN/../eridiffusion_amd' -Wl,-rpath,/opt/rocm/lib -Wl,-rpath,$(SANRT)

clean:
	rm -rf san_host _san

.PHONY: clean

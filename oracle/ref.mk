# Builds oracle/_ref/libref_torch.so from the REFERENCE's own torch-side sources where they lie (nothing is copied):
#   torchrec_embcache csrc: SwapManager, FeatureFilter (+ its logger);  hybrid_torchrec: IdsMapper, UniqueParallel.
# Needs the reference checkout and the installed PyTorch headers; used only to validate the CPU oracle.
REF ?= /root/reference
EMB := $(REF)/training/torch_rec_v1/torchrec_embcache/src/torchrec_embcache/csrc
HYB := $(REF)/training/torch_rec_v1/hybrid_torchrec/src/ids_process
PY ?= python3
TORCH_INC := $(shell $(PY) -c "from torch.utils.cpp_extension import include_paths; print(' '.join('-I'+p for p in include_paths()))")
TORCH_LIB := $(shell $(PY) -c "import torch,os; print(os.path.join(os.path.dirname(torch.__file__),'lib'))")
ABI := $(shell $(PY) -c "import torch; print(int(torch._C._GLIBCXX_USE_CXX11_ABI))")
CXX ?= g++
CXXFLAGS := -O1 -std=c++17 -fPIC -fopenmp -fvisibility=hidden -D_GLIBCXX_USE_CXX11_ABI=$(ABI) -w
SRCS := $(EMB)/embedding_cache/swap_manager.cpp $(EMB)/feature_filter/feature_filter.cpp \
        $(EMB)/feature_filter/evict_feature_record.cpp $(EMB)/utils/logger.cpp \
        $(HYB)/ids_mapper.cpp $(HYB)/unique.cpp ref_shim.cpp

_ref/libref_torch.so: ref_shim.cpp ref.mk
	mkdir -p _ref
	$(CXX) $(CXXFLAGS) -shared -o $@ $(SRCS) -I$(EMB) -I$(HYB) $(TORCH_INC) -L$(TORCH_LIB) -ltorch_cpu -ltorch -lc10 \
	    -Wl,-rpath,$(TORCH_LIB)

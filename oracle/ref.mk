# Compiles the part of the REFERENCE that builds from its own sources with gcc alone (deepxcore's
# IR parser, factory, dtype and shape-inference code, raw file I/O) into oracle/_ref/libdeepxref.so, from where the
# sources lie under $(REFERENCE).  Nothing is copied; outputs go to oracle/_ref/ only (git-ignored).
# Sections are garbage-collected so that functions needing the unbuildable parts (Shape's
# constructor lives in shape.cpp, which needs yaml-cpp) drop out instead of leaving undefined symbols.
# deepx/shape_matmul.cpp is left out for that reason: matmul_shape takes and returns Shape objects,
# whose constructors and operator[] are defined in shape.cpp, so nothing could call it.
REFERENCE ?= /root/reference
CORE := $(REFERENCE)/executor/deepxcore/src
CXX ?= g++
SRCS := $(CORE)/deepx/tf/tf.cpp $(CORE)/deepx/tf/tffactory.cpp $(CORE)/deepx/shape_changeshape.cpp \
        $(CORE)/deepx/shape_reduce.cpp $(CORE)/stdutil/num.cpp $(CORE)/stdutil/string.cpp $(CORE)/stdutil/fs.cpp
FLAGS := -O1 -std=c++17 -fPIC -w -fvisibility=hidden -ffunction-sections -fdata-sections -I$(CORE)

_ref/libdeepxref.so: ref_shim.cpp $(SRCS)
	mkdir -p _ref
	$(CXX) $(FLAGS) -shared -Wl,--gc-sections -Wl,-z,defs -o $@ ref_shim.cpp $(SRCS)

// model.cc — placeholder until the resident model lands (next commit).
#include "device.h"
extern "C" void rd_model_destroy(rd_model *) {}

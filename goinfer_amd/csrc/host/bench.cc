#include "device.h"

// Forwarding header: keeps the reference's include path working.
#pragma once
#include "gern/core/lang.h"

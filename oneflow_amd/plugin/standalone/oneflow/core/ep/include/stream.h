// Stand-alone build only: ep::Stream lives in the framework restatement.
#pragma once
#include "oneflow/core/framework/framework.h"

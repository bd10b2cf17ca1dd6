// Stand-alone build only: ep::Event lives in the framework restatement.
#pragma once
#include "oneflow/core/framework/framework.h"

// Umbrella header of the host layer (the subset of ginn/ginn.h that sits on
// or next to the matrix-product path).
#ifndef GINN_GINN_H
#define GINN_GINN_H

#include <ginn/autobatch.h>
#include <ginn/level_exec.h>
#include <ginn/def.h>
#include <ginn/dev.h>
#include <ginn/init/init.h>
#include <ginn/node.h>
#include <ginn/node/affine.h>
#include <ginn/node/common.h>
#include <ginn/node/compare.h>
#include <ginn/node/data.h>
#include <ginn/node/inplace.h>
#include <ginn/node/layernorm.h>
#include <ginn/node/layout.h>
#include <ginn/node/nlnode.h>
#include <ginn/node/pick.h>
#include <ginn/node/prod.h>
#include <ginn/node/reduce.h>
#include <ginn/node/select.h>
#include <ginn/node/weight.h>
#include <ginn/nonlin.h>
#include <ginn/prod.h>
#include <ginn/tensor.h>
#include <ginn/util/amax.h>
#include <ginn/util/util.h>

#endif  // GINN_GINN_H

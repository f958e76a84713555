// rt::NodesList under the file name the reference gives it (src/runtime/nodes-list.hh:10-24): the
// runner includes <nodes-list.hh>, and the include path picks this mirror or the reference's header.
#pragma once

#include "rt_graph.hh"

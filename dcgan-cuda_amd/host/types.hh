// Element type of every tensor on the path (reference: src/memory/types.hh:3).
#pragma once
using dbl_t = float;

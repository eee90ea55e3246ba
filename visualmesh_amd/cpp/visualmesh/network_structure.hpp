/* Forwarding header: the type lives in types.hpp; this file exists so that code written against the
 * reference's include layout (visualmesh/network_structure.hpp) compiles unchanged. */
#ifndef VISUALMESH_NETWORK_STRUCTURE_HPP
#define VISUALMESH_NETWORK_STRUCTURE_HPP
#include "types.hpp"
#endif

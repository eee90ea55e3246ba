/* Forwarding header: the type lives in types.hpp; this file exists so that code written against the
 * reference's include layout (visualmesh/projected_mesh.hpp) compiles unchanged. */
#ifndef VISUALMESH_PROJECTED_MESH_HPP
#define VISUALMESH_PROJECTED_MESH_HPP
#include "types.hpp"
#endif

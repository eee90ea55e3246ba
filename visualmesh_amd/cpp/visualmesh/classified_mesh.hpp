/* Forwarding header: the type lives in types.hpp; this file exists so that code written against the
 * reference's include layout (visualmesh/classified_mesh.hpp) compiles unchanged. */
#ifndef VISUALMESH_CLASSIFIED_MESH_HPP
#define VISUALMESH_CLASSIFIED_MESH_HPP
#include "types.hpp"
#endif

/* Forwarding header: fourcc() and fourcc_text() live in types.hpp; this file exists so that code written
 * against the reference's include layout (visualmesh/utility/fourcc.hpp) compiles unchanged. */
#ifndef VISUALMESH_UTILITY_FOURCC_HPP
#define VISUALMESH_UTILITY_FOURCC_HPP
#include "../types.hpp"
#endif

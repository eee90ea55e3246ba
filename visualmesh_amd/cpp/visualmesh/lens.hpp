/* Forwarding header: the type lives in types.hpp; this file exists so that code written against the
 * reference's include layout (visualmesh/lens.hpp) compiles unchanged. */
#ifndef VISUALMESH_LENS_HPP
#define VISUALMESH_LENS_HPP
#include "types.hpp"
#endif

/* Forwarding header: the type lives in types.hpp; this file exists so that code written against the
 * reference's include layout (visualmesh/node.hpp) compiles unchanged. */
#ifndef VISUALMESH_NODE_HPP
#define VISUALMESH_NODE_HPP
#include "types.hpp"
#endif

/*
 * Plain data types of the Visual Mesh engine interface.
 *
 * These are layout- and meaning-compatible with the reference's public types so that code written
 * against any of the reference engines compiles against visualmesh::engine::hip::Engine unchanged:
 *   Lens, LensProjection           reference lens.hpp:28-52
 *   Node                           reference node.hpp:39-45
 *   Layer, NetworkStructure, ...   reference network_structure.hpp:25-52
 *   ProjectedMesh                  reference projected_mesh.hpp:32-41
 *   ClassifiedMesh                 reference classified_mesh.hpp:37-48
 *   vec2/vec3/vec4/mat3/mat4       reference utility/math.hpp:27-40 (std::array aliases)
 *   fourcc, fourcc_text            reference utility/fourcc.hpp:34-46
 */
#ifndef VISUALMESH_TYPES_HPP
#define VISUALMESH_TYPES_HPP

#include <array>
#include <cstdint>
#include <string>
#include <vector>

namespace visualmesh {

template <typename Scalar>
using vec2 = std::array<Scalar, 2>;
template <typename Scalar>
using vec3 = std::array<Scalar, 3>;
template <typename Scalar>
using vec4 = std::array<Scalar, 4>;
template <typename Scalar>
using mat3 = std::array<vec3<Scalar>, 3>;
template <typename Scalar>
using mat4 = std::array<vec4<Scalar>, 4>;

enum LensProjection { RECTILINEAR, EQUISOLID, EQUIDISTANT };

template <typename Scalar>
struct Lens {
    std::array<int, 2> dimensions;    ///< image width and height in pixels
    LensProjection projection;        ///< projection model
    Scalar focal_length;              ///< in pixels
    std::array<Scalar, 2> centre;     ///< offset of the optical axis from the image centre
    std::array<Scalar, 2> k;          ///< radial distortion coefficients
    Scalar fov;                       ///< full field of view in radians
};

template <typename Scalar, int N_NEIGHBOURS>
struct Node {
    vec3<Scalar> ray;                          ///< unit vector in observation-plane space
    std::array<int, N_NEIGHBOURS> neighbours;  ///< absolute indices, clockwise; nodes.size() = no neighbour
};

template <typename Scalar>
using Weights = std::vector<std::vector<Scalar>>;
template <typename Scalar>
using Biases = std::vector<Scalar>;

enum ActivationFunction { SELU, RELU, SOFTMAX, TANH };

template <typename Scalar>
struct Layer {
    Weights<Scalar> weights;  ///< [inputs][outputs]
    Biases<Scalar> biases;    ///< [outputs]
    ActivationFunction activation;
};
template <typename Scalar>
using ConvolutionalGroup = std::vector<Layer<Scalar>>;
template <typename Scalar>
using NetworkStructure = std::vector<ConvolutionalGroup<Scalar>>;

template <typename Scalar, int N_NEIGHBOURS>
struct ProjectedMesh {
    std::vector<std::array<Scalar, 2>> pixel_coordinates;      ///< one per visible node
    std::vector<std::array<int, N_NEIGHBOURS>> neighbourhood;  ///< visible nodes + the null row
    std::vector<int> global_indices;                           ///< index of each visible node in the mesh
};

template <typename Scalar, int N_NEIGHBOURS>
struct ClassifiedMesh {
    std::vector<std::array<Scalar, 2>> pixel_coordinates;
    std::vector<std::array<int, N_NEIGHBOURS>> neighbourhood;
    std::vector<int> global_indices;
    std::vector<Scalar> classifications;  ///< (visible nodes + null row) x classes, row major
};

inline constexpr uint32_t fourcc(const char (&code)[5]) {
    return uint32_t(uint8_t(code[0])) | (uint32_t(uint8_t(code[1])) << 8) | (uint32_t(uint8_t(code[2])) << 16)
           | (uint32_t(uint8_t(code[3])) << 24);
}
inline std::string fourcc_text(const uint32_t& code) {
    return std::string({char(code & 0xFF), char(code >> 8 & 0xFF), char(code >> 16 & 0xFF), char(code >> 24 & 0xFF)});
}

}  // namespace visualmesh

#endif  // VISUALMESH_TYPES_HPP

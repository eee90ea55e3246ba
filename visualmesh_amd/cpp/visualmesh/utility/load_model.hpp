/*
 * Loading exported networks and dataset lens files without yaml-cpp
 * (reference example/load_model.hpp:25-52 and example/dataset.hpp:70-93; schema training/export.py:91-106).
 *
 *   auto network = visualmesh::load_model<float>("model.yaml");          // NetworkStructure<float>
 *   auto file    = visualmesh::load_model_file<float>("model.yaml");     // + mesh model name and geometry
 *   auto view    = visualmesh::load_lens<float>("lens0000000.yaml", w, h); // Lens + Hoc of one dataset element
 */
#ifndef VISUALMESH_UTILITY_LOAD_MODEL_HPP
#define VISUALMESH_UTILITY_LOAD_MODEL_HPP

#include <stdexcept>
#include <string>
#include <vector>

#include "../types.hpp"
#include "yaml_lite.hpp"

namespace visualmesh {

inline ActivationFunction activation_function(const std::string& name) {
    if (name == "selu") return ActivationFunction::SELU;
    if (name == "softmax") return ActivationFunction::SOFTMAX;
    if (name == "relu") return ActivationFunction::RELU;
    if (name == "tanh") return ActivationFunction::TANH;
    throw std::runtime_error("Unknown activation function " + name);
}

template <typename Scalar>
struct ModelFile {
    std::string mesh;             ///< mesh model name, e.g. "RING6"
    std::string shape;            ///< geometry shape name, e.g. "SPHERE"
    Scalar radius = 0;            ///< geometry radius
    Scalar intersections = 0;     ///< the number the exporter wrote under geometry.intersections
    NetworkStructure<Scalar> network;
};

template <typename Scalar>
NetworkStructure<Scalar> network_from_yaml(const yaml::Node& network) {
    NetworkStructure<Scalar> model;
    for (const yaml::Node& conv : network) {
        model.emplace_back();
        for (const yaml::Node& layer : conv) {
            Layer<Scalar> l;
            for (const yaml::Node& row : layer["weights"]) l.weights.push_back(row.template as_vector<Scalar>());
            l.biases = layer["biases"].template as_vector<Scalar>();
            l.activation = activation_function(layer["activation"].as_string());
            for (const auto& row : l.weights)
                if (row.size() != l.biases.size()) throw std::runtime_error("model: a weight row does not match the number of biases");
            model.back().push_back(std::move(l));
        }
    }
    return model;
}

template <typename Scalar>
ModelFile<Scalar> load_model_file(const std::string& path) {
    const yaml::Node config = yaml::load_file(path);
    ModelFile<Scalar> file;
    if (config.has("mesh")) file.mesh = config["mesh"].as_string();
    if (config.has("geometry")) {
        const yaml::Node& g = config["geometry"];
        if (g.has("shape")) file.shape = g["shape"].as_string();
        if (g.has("radius")) file.radius = static_cast<Scalar>(g["radius"].as_double());
        if (g.has("intersections")) file.intersections = static_cast<Scalar>(g["intersections"].as_double());
    }
    file.network = network_from_yaml<Scalar>(config["network"]);
    return file;
}

template <typename Scalar>
NetworkStructure<Scalar> load_model(const std::string& path) {
    return load_model_file<Scalar>(path).network;
}

template <typename Scalar>
struct LensFile {
    Lens<Scalar> lens;
    mat4<Scalar> Hoc;
};

/* the image dimensions are not in the file: the reference takes them from the image it loads next to it */
template <typename Scalar>
LensFile<Scalar> load_lens(const std::string& path, int width, int height) {
    const yaml::Node node = yaml::load_file(path);
    LensFile<Scalar> out;
    const std::string projection = node["projection"].as_string();
    if (projection == "RECTILINEAR") out.lens.projection = RECTILINEAR;
    else if (projection == "EQUIDISTANT") out.lens.projection = EQUIDISTANT;
    else if (projection == "EQUISOLID") out.lens.projection = EQUISOLID;
    else throw std::runtime_error("lens: unknown projection " + projection);
    out.lens.dimensions = {{width, height}};
    out.lens.focal_length = static_cast<Scalar>(node["focal_length"].as_double());
    const std::vector<Scalar> centre = node["centre"].template as_vector<Scalar>();
    const std::vector<Scalar> k = node["k"].template as_vector<Scalar>();
    if (centre.size() != 2 || k.size() != 2) throw std::runtime_error("lens: centre and k have two entries each");
    out.lens.centre = {{centre[0], centre[1]}};
    out.lens.k = {{k[0], k[1]}};
    out.lens.fov = static_cast<Scalar>(node["fov"].as_double());
    const yaml::Node& H = node["Hoc"];
    if (H.size() != 4) throw std::runtime_error("lens: Hoc has four rows");
    for (int r = 0; r < 4; ++r) {
        const std::vector<Scalar> row = H[r].template as_vector<Scalar>();
        if (row.size() != 4) throw std::runtime_error("lens: Hoc has four columns");
        for (int c = 0; c < 4; ++c) out.Hoc[r][c] = row[c];
    }
    return out;
}

}  // namespace visualmesh

#endif  // VISUALMESH_UTILITY_LOAD_MODEL_HPP

// Model files of the reference: the `.otter` network description (a block-structured text file) and the weight
// streams that go with it (Otter's own fp32 stream and ncnn's `.bin` with its per-tensor type tags). Same class
// names and call sequence as the reference, so that `net.load_otter(path, mode); net.load_weight(path, type)` reads
// a model exactly as it does there:
//
//   otter::core::Param / Otter / OtterLeader     Tensor/Otter.hpp:24-98, Tensor/Otter.cpp:12-258
//   otter::DataReader / DataReaderFromStdio      Tensor/DataReader.hpp:15-41, Tensor/DataReader.cpp
//   otter::InitializerFromDataReader             Tensor/Initializer.cpp:21-50
//   otter::InitializerNcnnFromDataReader         Tensor/Initializer.cpp:56-190
#ifndef OTTER_HIP_FILE_HPP
#define OTTER_HIP_FILE_HPP

#include <cstdio>
#include <istream>
#include <string>
#include <vector>

#include "otter_hip.hpp"

namespace otter {
namespace core {

// one `key: value` line
struct Param {
    Param(std::string type_, std::string info_) : type(std::move(type_)), info(std::move(info_)) {}
    std::string type;
    std::string info;
};

// one `Name { ... }` block: its own parameters and its nested blocks
class Otter {
public:
    explicit Otter(std::string name = "") : name_(std::move(name)) {}
    void setName(std::string name) { name_ = std::move(name); }
    void addParam(Param p) { params_.push_back(std::move(p)); }
    void addPartner(Otter o) { partners_.push_back(std::move(o)); }
    bool parseBlueprint(std::istream& blueprint);
    const std::string& getName() const { return name_; }
    // Tensor/Otter.cpp:85-95: the block's own parameters followed by those of every nested block, one level deep
    // (how the `Param { ... }` block of a layer reaches the layer's option table)
    std::vector<Param> getParams() const;
    const std::vector<Param>& ownParams() const { return params_; }
    const std::vector<Otter>& getPartners() const { return partners_; }
    bool idle() const { return params_.empty(); }

private:
    std::string name_;
    std::vector<Otter> partners_;
    std::vector<Param> params_;
};

// a whole file: `name: "..."`, file-level parameters, one block per layer
class OtterLeader {
public:
    explicit OtterLeader(std::string project_name = "") : project_name_(std::move(project_name)) {}
    const std::string& getProjectName() const { return project_name_; }
    size_t teams_size() const { return teams_.size(); }
    size_t params_size() const { return params_.size(); }
    const Otter& getTeam(int i) const { return teams_[i]; }
    const std::string& getTeamName(int i) const { return teams_[i].getName(); }
    std::vector<Param> getTeamParams(int i) const { return teams_[i].getParams(); }
    const std::vector<Param>& getParams() const { return params_; }
    bool readProject(const char* project_path);
    bool readProject(std::istream& project);

private:
    std::string project_name_;
    std::vector<Otter> teams_;
    std::vector<Param> params_;
};

}  // namespace core

class DataReader {
public:
    virtual ~DataReader() = default;
    virtual size_t read(void* buf, size_t size) const = 0;
    virtual size_t remain() const = 0;  // bytes left in the stream
};

class DataReaderFromStdio : public DataReader {
public:
    explicit DataReaderFromStdio(FILE* file) : file_(file) {}
    size_t read(void* buf, size_t size) const override;
    size_t remain() const override;

private:
    FILE* file_;
};

class DataReaderFromMemory : public DataReader {
public:
    DataReaderFromMemory(const void* data, size_t size) : p_((const unsigned char*)data), left_(size) {}
    size_t read(void* buf, size_t size) const override;
    size_t remain() const override { return left_; }

private:
    mutable const unsigned char* p_;
    mutable size_t left_;
};

// Otter's own weight stream: consecutive raw fp32 tensors
class InitializerFromDataReader : public Initializer {
public:
    explicit InitializerFromDataReader(const DataReader& dr) : dr_(dr) { type = InitializerType::Otter; }
    Tensor load(const std::vector<int64_t>& shape, int type) const override;

private:
    const DataReader& dr_;
};

// ncnn's `.bin`: a weight tensor (type 0) starts with a 4-byte tag -- 0x01306B47 fp16, 0x000D4B38 int8,
// 0x0002C056 raw fp32, 0 raw fp32, any other non-zero byte sum a 256-entry fp32 table followed by byte indices --
// and its payload is padded to a multiple of 4 bytes; type 1 tensors are raw fp32 without a tag
class InitializerNcnnFromDataReader : public Initializer {
public:
    explicit InitializerNcnnFromDataReader(const DataReader& dr) : dr_(dr) { type = InitializerType::Ncnn; }
    Tensor load(const std::vector<int64_t>& shape, int type) const override;

private:
    const DataReader& dr_;
};

}  // namespace otter

#endif

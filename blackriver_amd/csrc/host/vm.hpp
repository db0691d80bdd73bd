// The word machine: a small stack language in which the model is written.
//
// Source text is a stream of words.  Numbers and strings push themselves;
// `name @` reads a named value from the current hash, `value name !` stores
// one; `%def name ... %end` defines a user word; `[ a b c ]` pushes its items
// and then their count; everything else is a native word (C++ object with a
// run(Stack&) method) or a previously defined user word.  A program is first
// compiled to word codes, then linked into a flat DaG in which user words are
// expanded in place and every native word occurrence has its own object.
//
// Public types and their behaviour follow the reference machine
// (blackriver/dag.hpp:21-482, dag.cpp:43-556) closely enough that its model
// scripts (bloomz-7b/init.words, train.words) compile, link and run
// unchanged, and native words written against it (NativeWord, Stack,
// NWORD_CREATOR_DEFINE_LR, Enviroment::insert_native_word) plug in as they are.
#pragma once

#include <map>
#include <memory>
#include <string>
#include <variant>
#include <vector>

#include "common.hpp"

namespace br {

struct TensorType;
using tensor_t = std::shared_ptr<TensorType>;

// One value on the stack: a number, a string or a tensor handle.
struct Cell {
    enum CellType { T_Number, T_String, T_Tensor };
    const CellType type_;
    std::variant<double, const std::string, tensor_t> v_;

    Cell() : type_(T_Number), v_(0.0) {}
    Cell(double value) : type_(T_Number), v_(value) {}
    Cell(const std::string& value) : type_(T_String), v_(value) {}
    Cell(tensor_t value) : type_(T_Tensor), v_(value) {}

    bool is_number() const { return type_ == T_Number; }
    bool is_string() const { return type_ == T_String; }
    bool is_tensor() const { return type_ == T_Tensor; }
    const std::string& as_string() {
        br_assert(type_ == T_String, "Cell type can't convert to string!");
        return std::get<1>(v_);
    }
    double as_number() {
        br_assert(type_ == T_Number, "Cell type can't convert to number!");
        return std::get<0>(v_);
    }
    bool as_boolean() {
        br_assert(type_ == T_Number, "Cell type can't convert to boolean!");
        return std::get<0>(v_) != 0.0;
    }
    tensor_t as_tensor() {
        br_assert(type_ == T_Tensor, "Cell type can't convert to vector!");
        return std::get<2>(v_);
    }
};
std::ostream& operator<<(std::ostream& os, Cell& c);

struct Stack {
    size_t size() { return data_.size(); }
    void clear() { data_.clear(); }

    Cell& top() {
        need(1);
        return data_.back();
    }
    Cell pop() {
        need(1);
        Cell c = data_.back();
        data_.pop_back();
        return c;
    }
    void drop() {
        need(1);
        data_.pop_back();
    }
    void dup() { data_.push_back(top()); }
    // ( b a -- b a b a b a ): the pair is left three times over
    void dup2() {
        Cell a = pop(), b = pop();
        for (int i = 0; i < 3; i++) {
            data_.push_back(b);
            data_.push_back(a);
        }
    }
    // ( b a -- a b )
    void swap() {
        Cell a = pop(), b = pop();
        data_.push_back(a);
        data_.push_back(b);
    }
    // ( c b a -- b a c )
    void rot() {
        Cell a = pop(), b = pop(), c = pop();
        data_.push_back(b);
        data_.push_back(a);
        data_.push_back(c);
    }
    double pop_number() { return pop().as_number(); }
    // ( x1 .. xn n -- ) returned in source order
    std::vector<double> pop_number_list() {
        const size_t n = (size_t)pop_number();
        std::vector<double> out(n, 0.0);
        for (size_t i = 0; i < n; i++) out[n - 1 - i] = pop_number();
        return out;
    }
    const std::string pop_string() { return pop().as_string(); }
    tensor_t pop_tensor() { return pop().as_tensor(); }
    bool pop_boolean() { return pop().as_boolean(); }

    void push(Cell cell) { data_.push_back(cell); }
    void push_number(double n) { data_.push_back(Cell(n)); }
    void push_number_list(std::vector<double>& list) {
        for (double v : list) push_number(v);
        push_number((double)list.size());
    }
    void push_tensor(tensor_t t) { data_.push_back(Cell(t)); }
    void push_string(const std::string& s) { data_.push_back(Cell(s)); }

    std::vector<Cell> data_;

private:
    void need(size_t n) { br_assert(data_.size() >= n, "Can't access cell from empty stack!"); }
};
std::ostream& operator<<(std::ostream& os, Stack& stack);

// A namespace of named values.  An Enviroment owns several and `#` switches
// between them; the model scripts keep one set of weights per hash.
struct Hash {
    using Item = std::variant<double, std::string, tensor_t>;

    Item find(const std::string& name) {
        auto it = map_.find(name);
        if (it == map_.end()) {
            std::cout << "Find: " << name << std::endl;
            br_panic("Can't find value for name!");
        }
        return it->second;
    }
    bool has(const std::string& name) const { return map_.count(name) != 0; }
    double find_number(const std::string& name) { return std::get<0>(find(name)); }
    std::string find_string(const std::string& name) { return std::get<1>(find(name)); }
    tensor_t find_tensor(const std::string& name) { return std::get<2>(find(name)); }
    void set(const std::string& name, Item item) { map_[name] = item; }
    void drop(const std::string& name) { map_.erase(name); }

    static Cell Item2Cell(Item item) {
        if (item.index() == 0) return Cell(std::get<0>(item));
        if (item.index() == 1) return Cell(std::get<1>(item));
        return Cell(std::get<2>(item));
    }
    static Item Cell2Item(Cell& cell) {
        if (cell.is_number()) return Item(cell.as_number());
        if (cell.is_string()) return Item(cell.as_string());
        return Item(cell.as_tensor());
    }

private:
    std::map<std::string, Item> map_;
};

struct Enviroment;

// The five hash / namespace operators `@ ! !! # ##` need the environment.
struct BuiltinOperator {
    virtual ~BuiltinOperator() {}
    virtual void run(Enviroment* env) = 0;
};

// Everything else implemented in C++ only sees the stack.
struct NativeWord {
    virtual ~NativeWord() {}
    virtual void run(Stack& stack) = 0;
};
using NativeCreator = NativeWord*(Enviroment&);

// One compiled word: what the source said, before user words are expanded.
struct WordCode {
    enum Kind { Number, String, Builtin, Native, User } type_;
    std::string str_;
    double num_ = 0.0;
};
using UserWord = std::vector<WordCode>;
std::ostream& operator<<(std::ostream& os, const WordCode& c);

// A linked program: flat steps plus the word objects they refer to.
struct DaG {
    DaG() = delete;
    explicit DaG(Enviroment* env) : env_(env) {}
    ~DaG();
    DaG(const DaG&) = delete;
    DaG& operator=(const DaG&) = delete;

private:
    struct Step {
        enum Kind { PushNumber, PushString, RunBuiltin, RunNative, Skip } kind;
        double num;
        std::string str;
        size_t idx;
    };
    const Enviroment* env_;
    std::vector<Step> steps_;
    std::vector<NativeWord*> natives_;
    std::vector<BuiltinOperator*> builtins_;
    friend struct Enviroment;
};

struct Enviroment {
    explicit Enviroment(const int hash_num = 1);
    ~Enviroment();

    void insert_native_word(const std::string& name, NativeCreator* fn);
    // Registers a fusion: wherever a linked program runs the native words
    // `sequence` one after the other with nothing but operand pushes
    // (strings and `@`) and switches of the name scope (`n #`, which
    // neither touch a tensor nor leave anything on the stack: operands
    // already pushed are tensors, not names) in between, the earlier words are skipped -- their
    // operands simply stay on the stack -- and the last one is replaced by
    // `fused`, which pops the operands of the whole sequence (first word's
    // deepest) and must produce exactly what the sequence would have.
    void insert_fusion(const std::vector<std::string>& sequence, const std::string& fused);

    // compile + link; the caller owns the result and runs it with run()
    DaG* build(const std::string& txt);
    void run(DaG* dag);
    // compile + link + run once
    void execute(const std::string& txt);
    // compile + link, then list the flat program one step per entry:
    // "N:<number>", "S:<string>", "B:<builtin>", "W:<native word>"; with
    // `fused` the program is listed after the fusion pass that build() and
    // execute() apply ("-:<native word>" marks a word whose work moved into
    // the fused word that follows)
    std::vector<std::string> disassemble(const std::string& txt, bool fused = false);

    Stack& stack() { return stack_; }
    Hash& hash() { return hashes_[target_]; }
    void change(size_t new_hash);
    size_t hashes_current() { return target_; }
    size_t hashes_num() { return hashes_.size(); }

private:
    UserWord compile(const std::string& txt);
    void linking(DaG& dag, UserWord& word);
    void fuse(DaG& dag);
    void run_(DaG* dag);
    void load_base_words();

    std::map<std::string, UserWord> user_words_;
    std::map<std::string, NativeCreator*> native_words_;
    std::vector<std::pair<std::vector<std::string>, std::string>> fusions_;
    Stack stack_;
    std::vector<Hash> hashes_;
    size_t target_;
};

// Gives a NativeWord subclass the static `creator` that insert_native_word takes.
#define NWORD_CREATOR_DEFINE_LR(CLS)                   \
    static NativeWord* creator(Enviroment& env) {      \
        NativeWord* wd = new CLS();                    \
        return wd;                                     \
    }

}  // namespace br

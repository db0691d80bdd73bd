#include "vm.hpp"

#include <cctype>
#include <optional>
#include <sstream>

#include "runtime.hpp"
#include "tensor.hpp"

namespace br {

// ---------------------------------------------------------------- printing
std::ostream& operator<<(std::ostream& os, Cell& c) {
    if (c.is_string()) {
        os << "S:" << c.as_string();
    } else if (c.is_number()) {
        os << "N:" << std::fixed << c.as_number();
    } else {
        os << "T: (" << c.as_tensor()->to_string() << " )";
    }
    return os;
}

std::ostream& operator<<(std::ostream& os, const WordCode& c) {
    static const char* tag[] = {"N:", "S:", "B:", "NA:", "U:"};
    os << tag[c.type_];
    if (c.type_ == WordCode::Number)
        os << c.num_;
    else
        os << c.str_;
    return os;
}

std::ostream& operator<<(std::ostream& os, Stack& stack) {
    os << "----STACK(" << stack.size() << ")----" << std::endl;
    for (size_t i = 0; i < stack.data_.size(); i++) os << "==>" << i << " " << stack.data_[i] << std::endl;
    os << "----" << std::endl;
    return os;
}

// ---------------------------------------------------------------- scanning
namespace {

// Splits source text into raw tokens.  Separators are blanks and the purely
// cosmetic grouping characters ( ) { }; [ and ] are tokens of their own; a
// ';' outside a string starts a comment that runs to the end of the line; a
// string starts with " or ' , ends with the same character on the same line
// and keeps its quotes until classification.  (Tabs and carriage returns are
// accepted as blanks as well.)
std::vector<std::string> scan(const std::string& txt) {
    std::vector<std::string> out;
    std::string cur;
    char quote = 0;  // non-zero while inside a string
    auto flush = [&]() {
        if (!cur.empty()) {
            out.push_back(cur);
            cur.clear();
        }
    };
    const size_t n = txt.size();
    for (size_t i = 0; i < n; i++) {
        const char ch = txt[i];
        if (quote) {
            if (ch == '\n') br_panic("tokenize_line error, string must end in one line!");
            cur.push_back(ch);
            if (ch == quote) {
                out.push_back(cur);
                cur.clear();
                quote = 0;
            }
            continue;
        }
        switch (ch) {
            case '\n':
            case ' ':
            case '\t':
            case '\r':
            case '(':
            case ')':
            case '{':
            case '}':
                flush();
                break;
            case '[':
            case ']':
                flush();
                out.push_back(std::string(1, ch));
                break;
            case '"':
            case '\'':
                if (!cur.empty()) br_panic("tokenize_line error!");
                quote = ch;
                cur.push_back(ch);
                break;
            case ';':
                flush();
                while (i + 1 < n && txt[i + 1] != '\n') i++;
                break;
            default:
                cur.push_back(ch);
        }
    }
    if (quote) br_panic("tokenize_line error, string must end in one line!");
    flush();
    return out;
}

// A token that starts like a number is one: with '.' or 'e' it is parsed as a
// double, otherwise as an integer.
bool as_number(const std::string& tok, double& value) {
    const bool starts = isdigit((unsigned char)tok[0]) ||
                        (tok[0] == '-' && tok.size() >= 2 && isdigit((unsigned char)tok[1]));
    if (!starts) return false;
    if (tok.find('.') != std::string::npos || tok.find('e') != std::string::npos)
        value = atof(tok.c_str());
    else
        value = (double)atol(tok.c_str());
    return true;
}

bool reserved(const std::string& s) {
    return s == "true" || s == "false" || s == "null" || s == "@" || s == "!" || s == "!!" || s == "#" || s == "##";
}

// user word names: letters, digits and '_', not starting with a digit
bool valid_word_name(const std::string& s) {
    if (s.empty() || reserved(s) || isdigit((unsigned char)s[0])) return false;
    for (char ch : s)
        if (!(isalnum((unsigned char)ch) || ch == '_')) return false;
    return true;
}

WordCode make(WordCode::Kind k, const std::string& s = "", double n = 0.0) {
    WordCode c;
    c.type_ = k;
    c.str_ = s;
    c.num_ = n;
    return c;
}

}  // namespace

// --------------------------------------------------------------- compiling
UserWord Enviroment::compile(const std::string& txt) {
    const std::vector<std::string> tokens = scan(txt);

    UserWord main_code;
    std::optional<std::pair<std::string, UserWord>> def;  // the %def being collected
    std::optional<size_t> list_items;                      // inside [ ... ]
    auto sink = [&]() -> UserWord& { return def ? def->second : main_code; };

    for (size_t i = 0; i < tokens.size(); i++) {
        std::string tok = tokens[i];

        if (tok == "%def") {
            if (def) br_panic("Can't define a new user word inside another user word!");
            if (list_items) br_panic("Can't define a new user word inside a list macro!");
            if (++i >= tokens.size()) br_panic("Can't find #end for #def!");
            const std::string& name = tokens[i];
            if (!valid_word_name(name) || user_words_.count(name) || native_words_.count(name))
                br_panic("Can't a valid name for #def macro!");
            def = std::make_pair(name, UserWord());
            continue;
        }
        if (tok == "%end") {
            if (list_items) br_panic("Can't ending a word or in a list macro.");
            if (!def) br_panic("Find #end without #def");
            user_words_[def->first] = def->second;
            def.reset();
            continue;
        }
        if (tok == "[") {
            list_items = 0;
            continue;
        }
        if (tok == "]") {
            if (!list_items) br_panic("']' list macro appears without begin '['!");
            sink().push_back(make(WordCode::Number, "", (double)*list_items));
            list_items.reset();
            continue;
        }

        WordCode code;
        double number = 0.0;
        if (tok == "ture" || tok == "true") {  // the reference spells the literal "ture"
            code = make(WordCode::Number, "", 1.0);
        } else if (tok == "false") {
            code = make(WordCode::Number, "", 0.0);
        } else if (tok == "null") {
            code = make(WordCode::String, "");
        } else if (tok == "@" || tok == "!" || tok == "!!" || tok == "#" || tok == "##") {
            code = make(WordCode::Builtin, tok);
        } else if (tok[0] == '"' || tok[0] == '\'') {
            br_assert(tok.size() >= 2, " string must begin \" ' or $");
            br_assert(tok[0] == tok.back(), " string length wrong");
            code = make(WordCode::String, tok.substr(1, tok.size() - 2));
        } else if (tok[0] == '$') {
            code = make(WordCode::String, tok);  // the '$' stays part of the key
        } else if (as_number(tok, number)) {
            code = make(WordCode::Number, "", number);
        } else if (native_words_.count(tok)) {
            code = make(WordCode::Native, tok);
        } else if (user_words_.count(tok)) {
            code = make(WordCode::User, tok);
        } else {
            std::cout << tok << std::endl;
            br_panic("Find an invalid symbol is not string, number, builtin, user or native!");
        }
        if (list_items) list_items = *list_items + 1;
        sink().push_back(code);
    }
    if (list_items) br_panic("List macro without ']' ending!");
    if (def) br_panic("Define macro without #end ending!");
    return main_code;
}

// ---------------------------------------------------------------- builtins
namespace {

struct GetValue : public BuiltinOperator {  // name @  ->  value
    void run(Enviroment* env) override {
        const std::string name = env->stack().pop_string();
        env->stack().push(Hash::Item2Cell(env->hash().find(name)));
    }
};
struct SetValue : public BuiltinOperator {  // value name !
    void run(Enviroment* env) override {
        const std::string name = env->stack().pop_string();
        Cell cell = env->stack().pop();
        env->hash().set(name, Hash::Cell2Item(cell));
    }
};
struct DropValue : public BuiltinOperator {  // name !!
    void run(Enviroment* env) override { env->hash().drop(env->stack().pop_string()); }
};
struct SwitchHash : public BuiltinOperator {  // n #
    void run(Enviroment* env) override { env->change((size_t)env->stack().pop_number()); }
};
struct CurrentHash : public BuiltinOperator {  // ## -> n
    void run(Enviroment* env) override { env->stack().push_number((double)env->hashes_current()); }
};

BuiltinOperator* make_builtin(const std::string& sym) {
    if (sym == "@") return new GetValue();
    if (sym == "!") return new SetValue();
    if (sym == "!!") return new DropValue();
    if (sym == "#") return new SwitchHash();
    if (sym == "##") return new CurrentHash();
    br_panic("Find an unsupoorted builtin operator!");
}

}  // namespace

// ----------------------------------------------------------------- linking
DaG::~DaG() {
    for (auto* w : natives_) delete w;
    for (auto* b : builtins_) delete b;
}

void Enviroment::linking(DaG& dag, UserWord& word) {
    for (const WordCode& code : word) {
        DaG::Step step;
        step.num = 0.0;
        step.idx = 0;
        switch (code.type_) {
            case WordCode::Number:
                step.kind = DaG::Step::PushNumber;
                step.num = code.num_;
                dag.steps_.push_back(step);
                break;
            case WordCode::String:
                step.kind = DaG::Step::PushString;
                step.str = code.str_;
                dag.steps_.push_back(step);
                break;
            case WordCode::Builtin:
                step.kind = DaG::Step::RunBuiltin;
                step.str = code.str_;
                step.idx = dag.builtins_.size();
                dag.builtins_.push_back(make_builtin(code.str_));
                dag.steps_.push_back(step);
                break;
            case WordCode::Native: {
                auto it = native_words_.find(code.str_);
                if (it == native_words_.end()) br_panic("Call a un registered native word!");
                step.kind = DaG::Step::RunNative;
                step.str = code.str_;
                step.idx = dag.natives_.size();
                dag.natives_.push_back(it->second(*this));
                dag.steps_.push_back(step);
                break;
            }
            case WordCode::User: {
                auto it = user_words_.find(code.str_);
                if (it == user_words_.end()) br_panic("Call a un registered native word!");
                linking(dag, it->second);  // user words are expanded in place
                break;
            }
        }
    }
}

// ----------------------------------------------------------------- running
void Enviroment::run_(DaG* dag) {
    for (size_t pc = 0; pc < dag->steps_.size(); pc++) {
        const DaG::Step& s = dag->steps_[pc];
        switch (s.kind) {
            case DaG::Step::PushNumber: stack_.push_number(s.num); break;
            case DaG::Step::PushString: stack_.push_string(s.str); break;
            case DaG::Step::RunBuiltin: dag->builtins_[s.idx]->run(this); break;
            case DaG::Step::RunNative: dag->natives_[s.idx]->run(stack_); break;
            case DaG::Step::Skip: break;
            default: br_panic("Runing binary error can't bere!");
        }
    }
}

// The gradient lift is a setting of the (process-wide) computing context that
// scripts change with op.grad_lift; a new environment starts from "off", and
// one that goes away takes its setting with it.
static void reset_context_settings() {
    ComputingContext::grad_lift = 1.0f;
    ComputingContext::grad_lift_auto = false;
    ComputingContext::loss_head_overwrite = false;
}

Enviroment::Enviroment(const int hash_num) : target_(0) {
    hashes_.resize(hash_num > 0 ? (size_t)hash_num : 1);
    load_base_words();
    reset_context_settings();
}

Enviroment::~Enviroment() { reset_context_settings(); }

void Enviroment::insert_native_word(const std::string& name, NativeCreator* fn) {
    if (native_words_.count(name)) br_panic("Can't insert native word with same name!");
    native_words_[name] = fn;
}

void Enviroment::insert_fusion(const std::vector<std::string>& sequence, const std::string& fused) {
    br_assert(sequence.size() >= 2, "a fusion needs at least two words");
    br_assert(native_words_.count(fused) != 0, "the fused word must be registered first");
    fusions_.emplace_back(sequence, fused);
}

// Peephole pass over a linked program (see insert_fusion).
void Enviroment::fuse(DaG& dag) {
    auto is_push = [](const DaG::Step& s) {
        return s.kind == DaG::Step::PushString || (s.kind == DaG::Step::RunBuiltin && s.str == "@");
    };
    for (const auto& fusion : fusions_) {
        const std::vector<std::string>& seq = fusion.first;
        for (size_t i = 0; i < dag.steps_.size(); i++) {
            if (dag.steps_[i].kind != DaG::Step::RunNative || dag.steps_[i].str != seq[0]) continue;
            std::vector<size_t> at{i};
            size_t pc = i + 1;
            while (at.size() < seq.size() && pc < dag.steps_.size()) {
                const DaG::Step& s = dag.steps_[pc];
                if (s.kind == DaG::Step::RunNative && s.str == seq[at.size()]) {
                    at.push_back(pc);
                } else if (s.kind == DaG::Step::PushNumber && pc + 1 < dag.steps_.size() &&
                           dag.steps_[pc + 1].kind == DaG::Step::RunBuiltin && dag.steps_[pc + 1].str == "#") {
                    pc++;   // `n #`: a switch of the name scope
                } else if (!is_push(s)) {
                    break;
                }
                pc++;
            }
            if (at.size() != seq.size()) continue;
            for (size_t k = 0; k + 1 < at.size(); k++) dag.steps_[at[k]].kind = DaG::Step::Skip;
            DaG::Step& last = dag.steps_[at.back()];
            last.str = fusion.second;
            last.idx = dag.natives_.size();
            dag.natives_.push_back(native_words_[fusion.second](*this));
            i = at.back();
        }
    }
}

DaG* Enviroment::build(const std::string& txt) {
    std::unique_ptr<DaG> dag(new DaG(this));
    UserWord code = compile(txt);
    linking(*dag, code);
    fuse(*dag);
    return dag.release();
}

void Enviroment::run(DaG* dag) {
    br_assert(dag->env_ == this, "Can't be here!");
    run_(dag);
}

void Enviroment::execute(const std::string& txt) {
    DaG dag(this);
    UserWord code = compile(txt);
    linking(dag, code);
    fuse(dag);
    run_(&dag);
}

std::vector<std::string> Enviroment::disassemble(const std::string& txt, bool fused) {
    DaG dag(this);
    UserWord code = compile(txt);
    linking(dag, code);
    if (fused) fuse(dag);
    std::vector<std::string> out;
    for (const DaG::Step& s : dag.steps_) {
        std::ostringstream ss;
        switch (s.kind) {
            case DaG::Step::PushNumber: ss << "N:" << s.num; break;
            case DaG::Step::PushString: ss << "S:" << s.str; break;
            case DaG::Step::RunBuiltin: ss << "B:" << s.str; break;
            case DaG::Step::RunNative: ss << "W:" << s.str; break;
            case DaG::Step::Skip: ss << "-:" << s.str; break;
        }
        out.push_back(ss.str());
    }
    return out;
}

void Enviroment::change(size_t new_hash) {
    if (new_hash >= hashes_.size()) br_panic("Change hash out ot size");
    target_ = new_hash;
}

// -------------------------------------------------------------- base words
namespace {

#define BR_STACK_WORD(CLS, ...)                           \
    struct CLS : public NativeWord {                      \
        void run(Stack& stack) override { __VA_ARGS__; }  \
        NWORD_CREATOR_DEFINE_LR(CLS)                      \
    };

BR_STACK_WORD(WordDrop, stack.drop())
BR_STACK_WORD(WordDup, stack.dup())
BR_STACK_WORD(WordDup2, stack.dup2())
BR_STACK_WORD(WordSwap, stack.swap())
BR_STACK_WORD(WordRot, stack.rot())
BR_STACK_WORD(WordShow, std::cout << stack << std::endl)
BR_STACK_WORD(WordExit, exit(0))

// arithmetic on the two top numbers: ( b a -- b OP a )
template <typename F>
void binary(Stack& stack, F f) {
    const double a = stack.pop_number();
    const double b = stack.pop_number();
    stack.push_number(f(b, a));
}
BR_STACK_WORD(WordAdd, binary(stack, [](double b, double a) { return b + a; }))
BR_STACK_WORD(WordSub, binary(stack, [](double b, double a) { return b - a; }))
BR_STACK_WORD(WordMul, binary(stack, [](double b, double a) { return b * a; }))
BR_STACK_WORD(WordDiv, binary(stack, [](double b, double a) { return b / a; }))
BR_STACK_WORD(WordIntDiv, binary(stack, [](double b, double a) { return (double)(int)(b / a); }))

struct WordConcat : public NativeWord {  // ( b a -- "ba" )
    void run(Stack& stack) override {
        const std::string a = stack.pop_string();
        const std::string b = stack.pop_string();
        stack.push_string(b + a);
    }
    NWORD_CREATOR_DEFINE_LR(WordConcat)
};

struct WordEcho : public NativeWord {  // prints "<rank>:<seconds since boot>\t<msg>"
    void run(Stack& stack) override {
        const std::string msg = stack.pop_string();
        std::cout << CollectiveContext::mpi_rank << ":" << CollectiveContext::now() << "\t" << msg << std::endl;
    }
    NWORD_CREATOR_DEFINE_LR(WordEcho)
};

}  // namespace

void Enviroment::load_base_words() {
    insert_native_word("drop", WordDrop::creator);
    insert_native_word("dup", WordDup::creator);
    insert_native_word("dup2", WordDup2::creator);
    insert_native_word("swap", WordSwap::creator);
    insert_native_word("rot", WordRot::creator);
    insert_native_word("?", WordShow::creator);
    insert_native_word("^", WordExit::creator);
    insert_native_word("+", WordAdd::creator);
    insert_native_word("-", WordSub::creator);
    insert_native_word("*", WordMul::creator);
    insert_native_word("/", WordDiv::creator);
    insert_native_word("//", WordIntDiv::creator);
    insert_native_word("|", WordConcat::creator);
    insert_native_word("echo", WordEcho::creator);
}

}  // namespace br

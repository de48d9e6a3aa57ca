/*
 * Minimal command-line argument registry for the harness: long options (--name value), boolean flags,
 * integers with k/M/G suffixes (2^10, 2^20, 2^30), enumerations, defaults and range checks -- the part
 * of bpplib's ProgramArguments the reference's main() uses (experimental/k-means/k-means/k-means.cpp:295-338).
 */
#ifndef KMX_HOST_CLI_ARGS_HPP
#define KMX_HOST_CLI_ARGS_HPP

#include <cstdint>
#include <iostream>
#include <limits>
#include <map>
#include <set>
#include <stdexcept>
#include <string>
#include <vector>

class ArgumentException : public std::runtime_error
{
public:
	explicit ArgumentException(const std::string& what) : std::runtime_error(what) {}
};

class ProgramArguments
{
	enum class Kind { Int, Bool, String, Enum };
	struct Arg {
		Kind kind;
		std::string help;
		bool present = false;
		std::int64_t intValue = 0, minValue = 0, maxValue = std::numeric_limits<std::int64_t>::max();
		bool boolValue = false;
		std::string strValue;
		std::set<std::string> options;
	};
	std::map<std::string, Arg> mArgs;
	std::vector<std::string> mOrder;
	std::map<std::string, std::string> mAliases;
	std::vector<std::pair<std::string, std::string>> mConflicts;

	Arg& find(const std::string& name)
	{
		auto alias = mAliases.find(name);
		auto it = mArgs.find(alias == mAliases.end() ? name : alias->second);
		if (it == mArgs.end()) throw ArgumentException("Unknown argument '--" + name + "'.");
		return it->second;
	}
	const Arg& find(const std::string& name) const { return const_cast<ProgramArguments*>(this)->find(name); }

	static std::int64_t parseInt(const std::string& name, const std::string& text)
	{
		if (text.empty()) throw ArgumentException("Argument '--" + name + "' needs a number.");
		std::size_t pos = 0;
		std::int64_t value = 0;
		try { value = std::stoll(text, &pos); }
		catch (std::exception&) { throw ArgumentException("Argument '--" + name + "': '" + text + "' is not a number."); }
		std::string suffix = text.substr(pos);
		if (suffix == "k" || suffix == "K") value <<= 10;
		else if (suffix == "M") value <<= 20;
		else if (suffix == "G") value <<= 30;
		else if (!suffix.empty()) throw ArgumentException("Argument '--" + name + "': unknown suffix '" + suffix + "'.");
		return value;
	}

	Arg& add(const std::string& name, Kind kind, const std::string& help)
	{
		Arg a;
		a.kind = kind;
		a.help = help;
		mOrder.push_back(name);
		return mArgs[name] = a;
	}

public:
	void registerInt(const std::string& name, const std::string& help, std::int64_t def, std::int64_t min = 0,
		std::int64_t max = std::numeric_limits<std::int64_t>::max())
	{
		Arg& a = add(name, Kind::Int, help);
		a.intValue = def; a.minValue = min; a.maxValue = max;
	}
	void registerBool(const std::string& name, const std::string& help) { add(name, Kind::Bool, help); }
	void registerString(const std::string& name, const std::string& help, const std::string& def) { add(name, Kind::String, help).strValue = def; }
	void registerEnum(const std::string& name, const std::string& help, const std::string& def, std::initializer_list<std::string> options)
	{
		Arg& a = add(name, Kind::Enum, help);
		a.strValue = def;
		a.options = options;
	}
	void alias(const std::string& aliasName, const std::string& target) { mAliases[aliasName] = target; }
	void conflicts(const std::string& a, const std::string& b) { mConflicts.emplace_back(a, b); }

	void process(int argc, char** argv)
	{
		for (int i = 1; i < argc; ++i) {
			std::string token = argv[i];
			if (token.rfind("--", 0) != 0) throw ArgumentException("Unexpected token '" + token + "'.");
			std::string name = token.substr(2);
			Arg& a = find(name);
			a.present = true;
			if (a.kind == Kind::Bool) { a.boolValue = true; continue; }
			if (i + 1 >= argc) throw ArgumentException("Argument '--" + name + "' needs a value.");
			std::string value = argv[++i];
			if (a.kind == Kind::Int) {
				const std::int64_t parsed = parseInt(name, value);
				if (parsed < a.minValue || parsed > a.maxValue)
					throw ArgumentException("Argument '--" + name + "' is out of range [" + std::to_string(a.minValue) + ", " + std::to_string(a.maxValue) + "].");
				a.intValue = parsed;
			}
			else if (a.kind == Kind::Enum) {
				if (!a.options.count(value)) throw ArgumentException("Argument '--" + name + "': '" + value + "' is not one of the allowed values.");
				a.strValue = value;
			}
			else a.strValue = value;
		}
		for (auto& c : mConflicts)
			if (find(c.first).present && find(c.second).present)
				throw ArgumentException("Arguments '--" + c.first + "' and '--" + c.second + "' exclude each other.");
	}

	bool isPresent(const std::string& name) const { return find(name).present; }
	std::int64_t getInt(const std::string& name) const { return find(name).intValue; }
	bool getBool(const std::string& name) const { return find(name).boolValue; }
	const std::string& getString(const std::string& name) const { return find(name).strValue; }

	void printUsage(std::ostream& out) const
	{
		out << "Arguments:" << std::endl;
		for (auto& name : mOrder) {
			const Arg& a = mArgs.at(name);
			out << "  --" << name;
			if (a.kind == Kind::Int) out << " <int, default " << a.intValue << ">";
			else if (a.kind == Kind::String) out << " <string, default '" << a.strValue << "'>";
			else if (a.kind == Kind::Enum) {
				out << " <";
				bool first = true;
				for (auto& o : a.options) { out << (first ? "" : "|") << o; first = false; }
				out << ", default " << a.strValue << ">";
			}
			out << "  " << a.help << std::endl;
		}
	}
};

#endif

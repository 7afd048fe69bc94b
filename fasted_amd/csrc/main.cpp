// main.cpp -- command-line driver, the counterpart of main() in source/main.cu:143-186.
//
//   fasted -e <numPoints> <numDimensions> <epsilon>   seeded Exp(lambda=40) points in [0, 10]
//   fasted <file.csv> <epsilon>                       one point per line, comma separated
#include <cstring>
#include <iostream>
#include <stdexcept>
#include <string>

#include "../../include/fasted.h"

namespace {
double parse_double(const std::string& s) {
    try {
        return std::stod(s);
    } catch (const std::invalid_argument&) {
        throw std::invalid_argument("Invalid argument: unable to parse double");
    } catch (const std::out_of_range&) {
        throw std::out_of_range("Out of range: the number is too large or too small for a double");
    }
}
}  // namespace

int main(int argc, char* argv[]) {
    bool synthetic = false;
    for (int i = 1; i < argc; ++i)
        if (std::strcmp(argv[i], "-e") == 0) synthetic = true;

    if (synthetic) {
        if (argc != 5) {
            std::cerr << "Usage: " << argv[0] << " -e <numPoints> <numDimensions> <epsilon>" << std::endl;
            return 1;
        }
        const int numPoints = std::stoi(argv[2]);
        const int numDimensions = std::stoi(argv[3]);
        const double epsilon = parse_double(argv[4]);
        runFromExponentialDataset(numPoints, numDimensions, 40, 10.0, epsilon, false);
    } else {
        if (argc != 3) {
            std::cerr << "Usage: " << argv[0] << " <filename> <epsilon>" << std::endl;
            return 1;
        }
        runFromFile(argv[1], parse_double(argv[2]), false);
    }
    return 0;
}

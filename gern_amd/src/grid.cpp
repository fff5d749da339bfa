// Grid units, launch dimensions and the legality rules between them.
#include "gern/core/grid.h"
#include "gern/core/support.h"

namespace gern {

std::ostream &operator<<(std::ostream &os, const Grid::Unit &u) {
    static const char *names[] = {"UNDEFINED",         "SCALAR_UNIT",       "THREAD_X_IN_WRAPS", "THREAD_Y_IN_WRAPS",
                                  "THREAD_Z_IN_WRAPS", "THREAD_X",          "THREAD_Y",          "THREAD_Z",
                                  "WARP_X",            "WARP_Y",            "WARP_Z",            "BLOCK_X",
                                  "BLOCK_Y",           "BLOCK_Z"};
    const int i = (int)u;
    return os << ((i >= 0 && i < 14) ? names[i] : "UNDEFINED");
}

std::ostream &operator<<(std::ostream &os, const Grid::Dim &d) {
    static const char *names[] = {"GRID_DIM_X",  "GRID_DIM_Y", "GRID_DIM_Z", "BLOCK_DIM_X", "BLOCK_DIM_Y",
                                  "BLOCK_DIM_Z", "WARP_DIM_X", "WARP_DIM_Y", "WARP_DIM_Z",  "NULL_DIM"};
    const int i = (int)d;
    return os << ((i >= 0 && i < 10) ? names[i] : "NULL_DIM");
}

std::ostream &operator<<(std::ostream &os, const Grid::Level &l) {
    switch (l) {
    case Grid::Level::GRID:
        return os << "GRID";
    case Grid::Level::BLOCK_CLUSTER:
        return os << "BLOCK_CLUSTER";
    case Grid::Level::BLOCK:
        return os << "BLOCK";
    case Grid::Level::WARPS:
        return os << "WARPS";
    case Grid::Level::THREADS_WARPS:
        return os << "THREADS_WARPS";
    case Grid::Level::THREADS:
        return os << "THREADS";
    case Grid::Level::SCALAR:
        return os << "SCALAR";
    default:
        return os << "UNDEFINED";
    }
}

bool isLegalUnit(const Grid::Unit &u) {
    return u > Grid::Unit::SCALAR_UNIT;
}

bool isLegalLevel(const Grid::Level &l) {
    return l != Grid::Level::NULL_LEVEL;
}

Grid::Level getLevel(const Grid::Unit &u) {
    if (u == Grid::Unit::UNDEFINED) return Grid::Level::NULL_LEVEL;
    if (u == Grid::Unit::SCALAR_UNIT) return Grid::Level::SCALAR;
    if (u >= Grid::Unit::THREAD_X_IN_WRAPS && u <= Grid::Unit::THREAD_Z_IN_WRAPS) return Grid::Level::THREADS_WARPS;
    if (u >= Grid::Unit::THREAD_X && u <= Grid::Unit::THREAD_Z) return Grid::Level::THREADS;
    if (u >= Grid::Unit::WARP_X && u <= Grid::Unit::WARP_Z) return Grid::Level::WARPS;
    if (u >= Grid::Unit::BLOCK_X && u <= Grid::Unit::BLOCK_Z) return Grid::Level::BLOCK;
    return Grid::Level::SCALAR;
}

Grid::Level getLevel(const Grid::Dim &d) {
    if (d >= Grid::Dim::GRID_DIM_X && d <= Grid::Dim::GRID_DIM_Z) return Grid::Level::BLOCK;
    if (d >= Grid::Dim::BLOCK_DIM_X && d <= Grid::Dim::BLOCK_DIM_Z) return Grid::Level::THREADS;
    if (d >= Grid::Dim::WARP_DIM_X && d <= Grid::Dim::WARP_DIM_Z) return Grid::Level::THREADS_WARPS;
    return Grid::Level::NULL_LEVEL;
}

Grid::Level getLevel(const std::set<Grid::Unit> &units) {
    Grid::Level level = Grid::Level::NULL_LEVEL;
    for (const auto &u : units) {
        level = std::max(level, getLevel(u));
    }
    return level;
}

Grid::Level getLevel(const std::set<Grid::Dim> &dims) {
    Grid::Level level = Grid::Level::NULL_LEVEL;
    for (const auto &d : dims) {
        level = std::max(level, getLevel(d));
    }
    return level;
}

bool legalToDistribute(const std::set<Grid::Unit> &units, const Grid::Unit &over) {
    return isLegalUnit(over) && getLevel(units) <= getLevel(over);
}

Grid::Dim getDim(const Grid::Unit &u) {
    switch (u) {
    case Grid::Unit::THREAD_X:
    case Grid::Unit::WARP_X:
        return Grid::Dim::BLOCK_DIM_X;
    case Grid::Unit::THREAD_Y:
    case Grid::Unit::WARP_Y:
        return Grid::Dim::BLOCK_DIM_Y;
    case Grid::Unit::THREAD_Z:
    case Grid::Unit::WARP_Z:
        return Grid::Dim::BLOCK_DIM_Z;
    case Grid::Unit::THREAD_X_IN_WRAPS:
        return Grid::Dim::WARP_DIM_X;
    case Grid::Unit::THREAD_Y_IN_WRAPS:
        return Grid::Dim::WARP_DIM_Y;
    case Grid::Unit::THREAD_Z_IN_WRAPS:
        return Grid::Dim::WARP_DIM_Z;
    case Grid::Unit::BLOCK_X:
        return Grid::Dim::GRID_DIM_X;
    case Grid::Unit::BLOCK_Y:
        return Grid::Dim::GRID_DIM_Y;
    case Grid::Unit::BLOCK_Z:
        return Grid::Dim::GRID_DIM_Z;
    case Grid::Unit::UNDEFINED:
    case Grid::Unit::SCALAR_UNIT:
        return Grid::Dim::NULL_DIM;
    }
    throw error::UserError("Asking for the dim for an undefined unit!");
}

std::set<Grid::Dim> getDims(const std::set<Grid::Unit> &units) {
    std::set<Grid::Dim> dims;
    for (const auto &u : units) {
        dims.insert(getDim(u));
    }
    return dims;
}

bool isDimInScope(const Grid::Dim &dim, const std::set<Grid::Dim> &dims) {
    return dims.count(dim) > 0 || getLevel(dim) < getLevel(dims);
}

}  // namespace gern

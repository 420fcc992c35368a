// All weight containers (the reference's mat_type/mat_type.h).
#pragma once
#include "col_mat.hpp"
#include "csr_mat.h"
#include "mat1x16.h"
#include "row_mat.hpp"
#include "tile_mat.h"

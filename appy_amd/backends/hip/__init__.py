"""HIP C++ code generator and launcher for gfx950 (MI355X)."""

// Shadows fmt/core.h (not installed here); the data-structure sources compiled by the tests format nothing with it.
#pragma once

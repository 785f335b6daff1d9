"""MI355X-native K-FAC / Shampoo curvature path with the GradientMaker API of kazukiosawa/asdl."""

"""simple_knn package: `from simple_knn._C import distCUDA2`
(as imported at scene/gaussian_model.py:20 of CityGS-X)."""
